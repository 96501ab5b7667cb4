"""Oracle (test infrastructure): the per-layer KV-cache index state machine.

Follows wan/modules/causal_model.py:907-938 and 1102-1103 (index arithmetic, window
eviction, write-back of the two counters) and pipeline/causal_inference.py:288-303
(cache length: total_seq_len, or local_attn_size * tokens-per-frame).
Pure integer arithmetic; no tensors.
"""
from dataclasses import dataclass


@dataclass
class Step:
    """What one self-attention call does to the cache, in tokens."""
    roll_src: int          # eviction copy: cache[roll_src : roll_src+roll_len] -> cache[roll_dst : ...]
    roll_dst: int
    roll_len: int          # 0 when nothing is evicted
    cache_start: int       # the op sees cache[cache_start : cache_start + view_len]
    view_len: int
    write_start: int       # new K/V land at view[write_start : write_end]
    write_end: int


class KVCacheState:
    def __init__(self, cache_len, max_attention_size, frame_tokens, local_attn_size=-1, sink_frames=0):
        self.cache_len = cache_len
        self.max_attention_size = max_attention_size
        self.local_attn_size = local_attn_size
        self.sink_tokens = sink_frames * frame_tokens
        self.global_end = 0
        self.local_end = 0

    def step(self, current_start, num_new):
        current_end = current_start + num_new
        roll = (0, 0, 0)
        if (self.local_attn_size != -1 and current_end > self.global_end
                and num_new + self.local_end > self.cache_len):
            evicted = num_new + self.local_end - self.cache_len
            rolled = self.local_end - evicted - self.sink_tokens
            roll = (self.sink_tokens + evicted, self.sink_tokens, rolled)
            local_end = self.local_end + current_end - self.global_end - evicted
        else:
            local_end = self.local_end + current_end - self.global_end
        local_start = local_end - num_new
        cache_start = max(0, local_end - self.max_attention_size)
        st = Step(roll[0], roll[1], roll[2], cache_start, local_end - cache_start,
                  local_start - cache_start, local_end - cache_start)
        self.global_end = current_end
        # the reference stores the view-relative end (causal_model.py:937-938, 1103)
        self.local_end = local_end - cache_start
        return st
