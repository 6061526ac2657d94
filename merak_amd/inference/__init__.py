from .greedy import greedy_next_token, greedy_from_logits, DecodeStep
