from .greedy import greedy_next_token, greedy_from_logits, DecodeStep, top_k_logits, sample_next_token
from .llama_decode import LlamaDecoder, LlamaBlockWeights, rope_tables
