from .greedy import greedy_next_token, greedy_from_logits, DecodeStep, top_k_logits, sample_next_token
