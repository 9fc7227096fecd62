"""Legacy LlamaKVCache of the reference (src/kv_cache.rs:5-60) over the device cache."""
import numpy as np

from ._lib import check, lib
from .autograd import Tensor
from .layers import KVCacheInner


class LlamaKVCache:
    def __init__(self, config, ctx=None):  # kv_cache.rs:14-29
        self.max_seq_len = config.max_seq_len
        self.head_num = config.num_key_value_heads
        self.dim = config.hidden_size // config.num_attention_heads
        self._inner = KVCacheInner(1, self.head_num, self.max_seq_len, self.dim, ctx)

    def update(self, k, v, start_pos):  # kv_cache.rs:31-49, k/v [1, H_kv, S, D]
        s = k.shape[2]
        check(lib.lumen_kv_cache_update(self._inner.handle, k.ptr, v.ptr, s, start_pos))

    def get_view(self, current_len):  # kv_cache.rs:51-59: copies of the first current_len positions
        shape = (1, self.head_num, current_len, self.dim)
        kt = Tensor.empty(shape, np.float32, self._inner.ctx)
        vt = Tensor.empty(shape, np.float32, self._inner.ctx)
        check(lib.lumen_kv_cache_get_view(self._inner.handle, current_len, kt.ptr, vt.ptr))
        return kt, vt

    @property
    def k_cache(self):
        return self._inner.k

    @property
    def v_cache(self):
        return self._inner.v
