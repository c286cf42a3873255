"""Test-side helpers: build the same KV contents on the GPU (vTensor ranges) and on the host
(numpy arrays for the oracle), seeded and reproducible."""
from __future__ import annotations

import ctypes as C

import numpy as np

from oracle import oracle as O

CHUNK = 2 << 20


def round_up(x, m):
    return (x + m - 1) // m * m


def bf16_randn(rng, shape):
    return O.f32_to_bf16(rng.standard_normal(shape).astype(np.float32))


class GpuSeqs:
    """`num_slots` sequence slots of one layer, each with a K and a V range."""

    def __init__(self, vmm, num_slots, num_kv_heads, head_size, elem_bytes, max_tokens, layers=1, value_skew=0):
        self.vmm = vmm
        self.chunk = vmm.chunkBytes()  # CHUNK unless the pool was set up with larger chunks
        self.row_bytes = num_kv_heads * head_size * elem_bytes
        self.value_skew = value_skew  # bytes between the base of a V range and its first row (the engine uses 256)
        self.max_bytes = round_up(max_tokens * self.row_bytes + value_skew, self.chunk)
        self.segs = [vmm.KVcacheSegment(layers, self.max_bytes, 0, False) for _ in range(num_slots)]
        if value_skew:
            for seg in self.segs:
                seg.set_value_skew(value_skew)
        self.layers = layers
        self.k_tables = [vmm.KVCache(num_slots) for _ in range(layers)]
        self.v_tables = [vmm.KVCache(num_slots) for _ in range(layers)]
        vmm.copy_kv_cache(self.k_tables, self.v_tables, self.segs)

    def upload(self, slot, k_rows: np.ndarray, v_rows: np.ndarray, layer=0):
        """Write rows [T,Hkv,D] at offset 0 of the slot's ranges and set used size."""
        from glake_amd import _C

        seg = self.segs[slot]
        nbytes = k_rows.nbytes
        need = round_up(nbytes + self.value_skew, self.chunk) - seg.actual_size
        if need > 0:
            seg.expandMultiSegment(need // self.chunk)
        k_rows = np.ascontiguousarray(k_rows)
        v_rows = np.ascontiguousarray(v_rows)
        _C.check(_C.lib().vtkv_memcpy_h2d(seg.getKeyDevicePtr(layer), k_rows.ctypes.data_as(C.c_void_p), nbytes))
        _C.check(_C.lib().vtkv_memcpy_h2d(seg.getValueDevicePtr(layer), v_rows.ctypes.data_as(C.c_void_p), nbytes))
        seg.set_used_size(nbytes)

    def map_zeroed(self, nbytes, layer=0):
        """Map enough chunks for nbytes in every slot and clear them (fresh chunks hold stale data)."""
        from glake_amd import _C

        zeros = np.zeros(nbytes, np.uint8)
        for seg in self.segs:
            need = round_up(nbytes + self.value_skew, self.chunk) - seg.actual_size
            if need > 0:
                seg.expandMultiSegment(need // self.chunk)
            for dst in (seg.getKeyDevicePtr(layer), seg.getValueDevicePtr(layer)):
                _C.check(_C.lib().vtkv_memcpy_h2d(dst, zeros.ctypes.data_as(C.c_void_p), nbytes))

    def download(self, slot, nbytes, layer=0, which="k", dtype=np.uint8):
        from glake_amd import _C

        seg = self.segs[slot]
        out = np.empty(nbytes, np.uint8)
        src = seg.getKeyDevicePtr(layer) if which == "k" else seg.getValueDevicePtr(layer)
        _C.check(_C.lib().vtkv_memcpy_d2h(out.ctypes.data_as(C.c_void_p), src, nbytes))
        return out.view(dtype)

    def table_tensors(self, layer=0):
        """int64 device tensors of the per-slot base pointers (cache_engine.py:98-109)."""
        import torch

        k = torch.tensor([s.getKeyDevicePtr(layer) for s in self.segs], dtype=torch.int64, device="cuda")
        v = torch.tensor([s.getValueDevicePtr(layer) for s in self.segs], dtype=torch.int64, device="cuda")
        return k, v

    def close(self):
        for s in self.segs:
            s.destroy()
        for t in self.k_tables + self.v_tables:
            t.destroy()


def torch_bf16_from_bits(bits: np.ndarray, device="cuda"):
    import torch

    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).to(device)


def bits_from_torch_bf16(t) -> np.ndarray:
    import torch

    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
