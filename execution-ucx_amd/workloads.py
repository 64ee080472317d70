"""Synthetic bundles used by the benchmark and the parity tests.

Every generator is seeded and returns a plain description (numpy only); the
``materialize_*`` helpers place it in device memory with torch, which is used
here for allocation and random fill only.

C1  64 contiguous fp32 tensors of 16,384 elements, uniform[-1, 1), host memory
C2  4,096 1-D tensors, sizes log-uniform 256 B..64 KiB rounded to the element
    size, dtypes cycled fp16/bf16/fp32/int32/int8, random bit patterns,
    256-byte aligned pack offsets
C3  one Llama-7B layer in bf16: q/k/v/o 4096x4096, gate/up 11008x4096,
    down 4096x11008, two RMSNorm vectors of 4096
C4  KV cache [layers, 2, blocks, 16, 8, 128] bf16; gather `picks` seeded block
    indices across all layers as strided views, scatter at another permutation
C5  streamed chunks, each built from 64 strided 2-D views with a row pitch of
    1.5x the row length
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence, Tuple

import numpy as np

from .dlpack import TensorView, kDLBfloat, kDLFloat, kDLInt
from . import _capi

# (name, DLPack dtype triple, bytes per element)
C2_DTYPES = [
    ("float16", (kDLFloat, 16, 1), 2),
    ("bfloat16", (kDLBfloat, 16, 1), 2),
    ("float32", (kDLFloat, 32, 1), 4),
    ("int32", (kDLInt, 32, 1), 4),
    ("int8", (kDLInt, 8, 1), 1),
]


@dataclass
class Segment:
    dtype: Tuple[int, int, int]
    dtype_name: str
    nbytes: int
    arena_offset: int   # where the tensor starts inside the source arena


@dataclass
class MixedBundle:
    """C2-style bundle: many 1-D tensors carved out of one byte arena."""
    segments: List[Segment]
    arena_bytes: int
    data_bytes: int


def mixed_bundle(n: int = 4096, lo: int = 256, hi: int = 65536, seed: int = 0,
                 gap_unit: int = 16, max_gap_units: int = 16) -> MixedBundle:
    rng = np.random.default_rng(seed)
    raw = np.exp(rng.uniform(np.log(lo), np.log(hi), size=n))
    gaps = rng.integers(0, max_gap_units, size=n) * gap_unit
    segs = []
    at = 0
    total = 0
    for i in range(n):
        name, dl, item = C2_DTYPES[i % len(C2_DTYPES)]
        nb = max(item, int(raw[i]) // item * item)
        at += int(gaps[i])
        at = (at + 15) // 16 * 16
        segs.append(Segment(dl, name, nb, at))
        at += nb
        total += nb
    return MixedBundle(segs, (at + 255) // 256 * 256, total)


LLAMA7B_LAYER = [
    ("q_proj", (4096, 4096)), ("k_proj", (4096, 4096)), ("v_proj", (4096, 4096)),
    ("o_proj", (4096, 4096)), ("gate_proj", (11008, 4096)), ("up_proj", (11008, 4096)),
    ("down_proj", (4096, 11008)), ("input_layernorm", (4096,)),
    ("post_attention_layernorm", (4096,)),
]


def llama_layer_bytes() -> int:
    return sum(int(np.prod(s)) * 2 for _, s in LLAMA7B_LAYER)


def host_bundle_c1(seed: int = 0, n: int = 64, elems: int = 16384) -> List[np.ndarray]:
    rng = np.random.default_rng(seed)
    return [rng.uniform(-1.0, 1.0, size=elems).astype(np.float32) for _ in range(n)]


@dataclass
class KvGather:
    layers: int
    blocks: int
    block_shape: Tuple[int, int, int]   # (tokens, heads, dim)
    src_index: np.ndarray
    dst_index: np.ndarray

    @property
    def cache_shape(self):
        return (self.layers, 2, self.blocks) + self.block_shape

    @property
    def block_elems(self):
        return int(np.prod(self.block_shape))

    @property
    def payload_bytes(self):
        return len(self.src_index) * self.layers * 2 * self.block_elems * 2


def kv_gather(layers: int = 32, blocks: int = 4096, picks: int = 512, seed: int = 0,
              block_shape=(16, 8, 128)) -> KvGather:
    rng = np.random.default_rng(seed)
    src = rng.choice(blocks, size=picks, replace=False)
    dst = np.random.default_rng(seed + 1).choice(blocks, size=picks, replace=False)
    return KvGather(layers, blocks, tuple(block_shape), src, dst)


def kv_block_view(base_ptr: int, spec: KvGather, block: int, device_id: int = 0) -> TensorView:
    """cache[:, :, block] as a strided view: shape [layers, 2, T, H, D]."""
    t, h, d = spec.block_shape
    be = spec.block_elems
    shape = (spec.layers, 2, t, h, d)
    strides = (2 * spec.blocks * be, spec.blocks * be, h * d, d, 1)
    return TensorView(data=base_ptr + block * be * 2, device_type=_capi.kDLROCM,
                      device_id=device_id, dtype=(kDLBfloat, 16, 1), shape=shape, strides=strides)


@dataclass
class PitchedChunk:
    views: int
    rows: int
    cols: int
    pitch: int   # elements

    @property
    def view_bytes(self):
        return self.rows * self.cols * 2

    @property
    def payload_bytes(self):
        return self.views * self.view_bytes

    @property
    def parent_elems(self):
        return self.rows * self.pitch


def pitched_chunk(views: int = 64, rows: int = 1024, cols: int = 2048) -> PitchedChunk:
    return PitchedChunk(views, rows, cols, cols * 3 // 2)


def pitched_views(base_ptr: int, spec: PitchedChunk, device_id: int = 0) -> List[TensorView]:
    """`views` parents of [rows, pitch] bf16 laid back to back from base_ptr;
    each view is parent[:, :cols]."""
    out = []
    for v in range(spec.views):
        out.append(TensorView(data=base_ptr + v * spec.parent_elems * 2,
                              device_type=_capi.kDLROCM, device_id=device_id,
                              dtype=(kDLBfloat, 16, 1), shape=(spec.rows, spec.cols),
                              strides=(spec.pitch, 1)))
    return out


# ---------------------------------------------------------------- torch side

def torch_dtype(name: str):
    import torch
    return getattr(torch, name)


def materialize_mixed(bundle: MixedBundle, device: str = "cuda", seed: int = 0):
    """Returns (arena uint8 tensor, list of typed 1-D tensor views)."""
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    arena = torch.randint(0, 256, (bundle.arena_bytes,), dtype=torch.uint8, device=device,
                          generator=g)
    tensors = []
    for s in bundle.segments:
        piece = arena[s.arena_offset:s.arena_offset + s.nbytes]
        tensors.append(piece.view(torch_dtype(s.dtype_name)))
    return arena, tensors


def mixed_views(bundle: MixedBundle, arena_ptr: int, device_id: int = 0,
                device_type: int = _capi.kDLROCM) -> List[TensorView]:
    """The same tensors described directly (no per-tensor DLPack round trip)."""
    out = []
    for s in bundle.segments:
        item = (s.dtype[1] + 7) // 8
        out.append(TensorView(data=arena_ptr + s.arena_offset, device_type=device_type,
                              device_id=device_id, dtype=s.dtype, shape=(s.nbytes // item,),
                              strides=None))
    return out


def materialize_llama_layer(device: str = "cuda", seed: int = 0):
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    out = []
    for _, shape in LLAMA7B_LAYER:
        t = torch.empty(shape, dtype=torch.float32, device=device)
        t.normal_(0.0, 0.02, generator=g)
        out.append(t.to(torch.bfloat16))
    return out


def views_of_torch(tensors: Sequence) -> List[TensorView]:
    """TensorViews of torch tensors without going through DLPack capsules."""
    import torch
    code = {torch.float16: (kDLFloat, 16, 1), torch.bfloat16: (kDLBfloat, 16, 1),
            torch.float32: (kDLFloat, 32, 1), torch.float64: (kDLFloat, 64, 1),
            torch.int32: (kDLInt, 32, 1), torch.int8: (kDLInt, 8, 1), torch.int16: (kDLInt, 16, 1),
            torch.int64: (kDLInt, 64, 1), torch.uint8: (1, 8, 1), torch.bool: (6, 8, 1),
            torch.complex64: (5, 64, 1), torch.complex128: (5, 128, 1)}
    out = []
    for t in tensors:
        dev = _capi.kDLROCM if t.is_cuda else _capi.kDLCPU
        out.append(TensorView(data=t.data_ptr(), device_type=dev,
                              device_id=t.device.index or 0, dtype=code[t.dtype],
                              shape=tuple(t.shape), strides=tuple(t.stride()), owner=t))
    return out
