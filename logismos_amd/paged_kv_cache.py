"""Host-side mirror of the `KvCache` trait (crates/cache/src/lib.rs:57-82) over the paged
device cache of the C-ABI library: `put`, `get`, `len_of`, `num_layers`, `reset` keep the
trait's names and meaning, per sequence; errors carry the names of the reference's
`cache::Error` variants (crates/cache/src/error.rs)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import hip, kernels


class CacheError(RuntimeError):
    KINDS = {1: "LayerOutOfRange", 2: "LenOverflow", 3: "ReadBeyondWritten", 4: "ShapeMismatch",
             5: "BadSeq", 6: "OutOfBlocks", 7: "OutOfSeqs", 8: "Hip"}

    def __init__(self, op: str, code: int):
        self.op, self.code, self.kind = op, int(code), self.KINDS.get(int(code), "Unknown")
        super().__init__(f"cache: {op}: {self.kind} (code {self.code})")


def _check(op: str, code: int) -> None:
    if code != 0:
        raise CacheError(op, code)


class PagedKvCache:
    def __init__(self, num_layers: int, num_kv_heads: int, head_dim: int, block_size: int,
                 num_blocks: int, max_seqs: int, max_blocks_per_seq: int):
        self._lib = kernels.library()
        self.layout = kernels.PagedKvLayout(num_layers, num_kv_heads, head_dim, block_size,
                                            num_blocks, max_seqs, max_blocks_per_seq)
        self._h = C.c_void_p()
        _check("create", self._lib.logismos_paged_kv_cache_create(C.byref(self.layout),
                                                                  C.byref(self._h)))

    def close(self) -> None:
        if self._h:
            self._lib.logismos_paged_kv_cache_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- the trait
    def put(self, seq_id: int, layer_idx: int, k, v, n_tokens: int, stream=None) -> None:
        _check("put", self._lib.logismos_paged_kv_cache_put(
            self._h, seq_id, layer_idx, kernels._ptr(k), kernels._ptr(v), n_tokens,
            kernels._raw(stream)))

    def get(self, seq_id: int, layer_idx: int, length: int, stream=None):
        """First `length` rows of (seq, layer) as two fp16 arrays [length][kv_heads*head_dim]."""
        row = self.layout.num_kv_heads * self.layout.head_dim
        k = hip.DeviceBuffer(max(16, length * row * 2))
        v = hip.DeviceBuffer(max(16, length * row * 2))
        _check("get", self._lib.logismos_paged_kv_cache_get(
            self._h, seq_id, layer_idx, length, k.ptr, v.ptr, kernels._raw(stream)))
        (stream.synchronize() if stream else hip.synchronize())
        return (k.to_numpy(np.float16, (length, row)), v.to_numpy(np.float16, (length, row)))

    def len_of(self, seq_id: int, layer_idx: int):
        n = self._lib.logismos_paged_kv_cache_len_of(self._h, seq_id, layer_idx)
        return None if n < 0 else int(n)

    def num_layers(self) -> int:
        return self._lib.logismos_paged_kv_cache_num_layers(self._h)

    def reset(self) -> None:
        self._lib.logismos_paged_kv_cache_reset(self._h)

    # ---- sequences and blocks
    def open_seq(self) -> int:
        s = C.c_int(-1)
        _check("open_seq", self._lib.logismos_paged_kv_cache_open_seq(self._h, C.byref(s)))
        return s.value

    def close_seq(self, seq_id: int) -> None:
        _check("close_seq", self._lib.logismos_paged_kv_cache_close_seq(self._h, seq_id))

    def reserve(self, seq_id: int, total_rows: int, stream=None) -> None:
        _check("reserve", self._lib.logismos_paged_kv_cache_reserve(self._h, seq_id, total_rows,
                                                                    kernels._raw(stream)))

    def advance(self, seq_id: int, layer_idx: int, n_tokens: int) -> None:
        _check("advance", self._lib.logismos_paged_kv_cache_advance(self._h, seq_id, layer_idx,
                                                                    n_tokens))

    def free_blocks(self) -> int:
        return self._lib.logismos_paged_kv_cache_free_blocks(self._h)

    def k_pool(self, layer_idx: int) -> C.c_void_p:
        return C.c_void_p(self._lib.logismos_paged_kv_cache_k_pool(self._h, layer_idx))

    def v_pool(self, layer_idx: int) -> C.c_void_p:
        return C.c_void_p(self._lib.logismos_paged_kv_cache_v_pool(self._h, layer_idx))

    def block_tables(self) -> C.c_void_p:
        return C.c_void_p(self._lib.logismos_paged_kv_cache_block_tables(self._h))

    def block_tables_host(self) -> np.ndarray:
        p = self._lib.logismos_paged_kv_cache_block_tables_host(self._h)
        n = self.layout.max_seqs * self.layout.max_blocks_per_seq
        a = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_int32)), shape=(n,))
        return a.reshape(self.layout.max_seqs, self.layout.max_blocks_per_seq).copy()
