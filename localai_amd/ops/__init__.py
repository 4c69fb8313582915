"""Operator layer: HIP (gfx950) kernels via a C ABI, plus fp32 PyTorch references.

Dispatch rule: a tensor on a GPU runs the hand-written HIP kernel from
`_la_kernels.so` -- there is NO silent eager fallback on the GPU (a missing library
raises).  CPU tensors run the PyTorch reference, which is also the numerics oracle
for the GPU tests (tests/test_kernels_gpu.py).

Every wrapper validates shapes/dtypes/contiguity on the host before launching, so a
bad call fails in Python instead of faulting the device.
"""
from __future__ import annotations

import ctypes
import functools
import math
import os
import threading
import warnings
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..gguf import GGMLType, dequantize

_LIB = None
_LIB_LOCK = threading.Lock()

FMT_Q8_0, FMT_Q4_K, FMT_Q6_K, FMT_BF16 = 8, 12, 14, 30
FMT_F32 = 0   # dense fp32 [N, K] (models served in true 32-bit: library SGEMM, no reduced-precision mode)


_REQUIRED: Optional[Tuple[str, ...]] = None


def require_kernels(files: Optional[Sequence[str]]) -> None:
    """Before the first lib(): the kernel sources this process will launch (a model class's
    `kernel_sources`).  Where the whole library is built it is loaded as always; on a checkout
    without it only these sources are compiled (ops/_build.build_subset) instead of every GEMM
    family.  None: no restriction."""
    global _REQUIRED
    _REQUIRED = tuple(sorted(set(files))) if files else None


def lib():
    """Load (building if needed) the kernel library.  Raises if unavailable."""
    global _LIB
    if _LIB is not None:
        return _LIB
    with _LIB_LOCK:
        if _LIB is not None:
            return _LIB
        from . import _build
        path = _build.LIB
        alt = os.environ.get("LOCALAI_AMD_KLIB")  # an A/B build of the same sources (_build.build_variant)
        partial = False
        if alt:
            path = _build.HERE / alt
        elif not path.exists() and _REQUIRED and not os.environ.get("LOCALAI_AMD_REBUILD"):
            path = _build.build_subset(_REQUIRED)
            partial = True
        elif not path.exists() or os.environ.get("LOCALAI_AMD_REBUILD"):
            _build.build()
        L = ctypes.CDLL(str(path))
        P, I, F, LNG = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_long
        sig = {
            "la_qgemm_skinny": [I, P, P, P, P, I, I, P, I, I, I, P, I, LNG, P],
            "la_qgemv_dp4": [I, P, P, P, I, P, I, I, I, P, I, LNG, P, LNG, I, P, I, P],
            "la_moe_gemv": [I, I, P, I, I, I, P, I, I, P, I, I, P, LNG, I, I, P, P, I, LNG, P],
            "la_gemv_variant": [I],
            "la_moe_tune": [I, I],
            "la_dec_one_part": [I],
            "la_gather_rows": [P, P, LNG, P, P, LNG, P],
            "la_qgemv_dp4_rope": [I, P, P, P, I, P, I, P, P, P, I, I, I, P, P, P, I, P],
            "la_qgemv_dp4_norm": [I, P, P, P, I, I, I, P, I, LNG, P, P, LNG, I, P, P, F, P, P],
            "la_qgemv_dp4_rope_norm": [I, P, P, P, I, I, P, P, P, I, I, I, P, P, P, I, P, P, LNG, I, P, P, F,
                                       P, P],
            "la_add_norm": [P, P, LNG, I, P, I, P, P, P, I, I, F, I, P, P],
            "la_add_norm_router": [P, P, LNG, I, P, I, P, P, P, I, I, F, I, P, I, I, I, F, I, I, P, P, P],
            "la_rope_kv": [P, LNG, I, P, P, P, P, I, I, I, I, I, I, P, P, P, I, P],
            "la_mamba_conv_step": [P, P, LNG, P, P, P, I, I, I, P],
            "la_groupnorm_nhwc": [P, P, P, P, P, I, I, I, I, I, I, F, I, P],
            "la_mamba_ssm_step": [P, P, P, P, LNG, I, I, P, P, P, LNG, P, I, I, I, P],
            "la_act": [P, LNG, I, P, P, I, I, I, P],
            "la_reduce_slabs": [P, LNG, I, P, I, I, P, P, P],
            "la_embed": [I, P, P, P, P, I, I, P, I, P, F, P],
            "la_dequant": [I, P, P, P, P, I, I, P, P],
            "la_attn_decode": [P, P, P, P, I, P, I, I, I, I, I, F, I, I, P, P, P, P, P, LNG, I, P, P, P, P, F, I, I, P, I, P,
                               P],
            "la_attn_prefill": [P, P, P, P, I, P, P, P, I, I, I, I, I, F, P, F, I, P, I, P, P],
            "la_sample": [P, LNG, I, I, P, P, P, P, P],
            "la_penalties": [P, LNG, I, P, I, P, P, I, P, P],
            "la_penalties_cols": [P, LNG, I, P, I, P, P, I, P, I, I, P],
            "la_tp_topc": [P, LNG, I, I, I, I, P, P],
            "la_tp_mirostat": [I, P, LNG, I, I, I, I, I, P, P, P, P, P, P, P, P],
            "la_grammar_mask": [P, LNG, I, I, P, P, LNG, P],
            "la_grammar_advance": [P, P, P, I, I, P],
            "la_sample_row_bytes": [],
            "la_logit_bias": [P, LNG, P, P, P, P, I, P],
            "la_moe_route": [P, I, I, I, P, P, P],
            "la_moe_router": [P, I, P, I, I, I, I, I, F, I, I, P, P, P],
            "la_moe_gemm": [I, I, P, I, I, I, P, P, I, P, I, I, I, P, P, I, LNG, I, P],
            "la_qw_size": [],
            "la_gemm_scales": [I, P, P, I, I, P, P],
            "la_qgemm_tile": [I, P, P, P, I, I, P, I, I, I, P, I, LNG, I, I, I, P],
            "la_qgemm_tile_probe": [P, P, I, I, P, I, I, P, I, I, P],
            "la_qgemm_tile2": [I, P, P, P, I, I, P, P, P, I, I, P, I, I, I, P, I, LNG, I, I, P],
            "la_pen_push": [P, I, P, I, P, P, P, P],
            "la_qgemm_glu": [I, P, P, P, I, P, P, P, I, I, I, P, I, I, P, I, I, I, P],
            "la_qgemm32": [I, P, P, P, I, I, P, I, I, I, P, I, LNG, I, I, P],
            "la_moe32": [I, I, P, I, I, I, P, P, I, P, I, I, I, P, P, I, LNG, I, I, P],
            "la_moe32_probe": [I, P, I, I, I, P, P, I, P, I, I, P, I, P],
            "la_qgemm32_2": [I, P, P, P, I, I, P, P, P, I, I, P, I, I, I, P, I, LNG, I, I, P],
            "la_qgemm32_glu": [I, P, P, P, I, P, P, P, I, I, I, P, I, I, P, I, I, I, P],
            "la_qgemm32_probe": [I, I, P, P, I, I, P, I, I, P, P],
            "la_attn_dense": [P, LNG, P, LNG, P, LNG, P, LNG, P, I, P, I, I, I, F, P],
            "la_bsgemm": [I, P, P, P, I, I, P, I, I, I, P, I, LNG, I, I, P],
            "la_bsgemm2": [I, P, P, P, I, I, P, P, P, I, I, P, I, I, I, P, I, LNG, I, I, P],
            "la_bsgemm_glu": [I, P, P, P, I, P, P, P, I, I, I, P, I, I, P, I, I, I, P],
            "la_bsmoe": [I, I, P, I, I, I, P, P, I, P, I, I, I, P, P, I, LNG, I, I, P],
            "la_decode_advance": [P, P, P, P, P, P, I, I, I, P, I, P, P, P],
            "la_shortconv_kv": [I, I, P, I, P, P, I, I, I, I, P, P, P, P, P, P, P, P, P, I, I, I, I, P, P, P, I, I, P],
            "la_attn_mix_rows": [I, P, P, P, P, P, P, I, I, I, I, I, I, I, F, F, P, P, I, I, P, I, P, P, I, P, P],
            "la_attn_mix_tiles": [P, P, P, P, I, P, P, P, I, I, I, I, I, I, F, F, P, P, I, I, P, I, P, I, P, P, I, P, I, P,
                                  P],
            "la_router_sigmoid": [I, P, LNG, P, P, I, I, I, I, I, P, P, P],
            "la_router_topk": [I, I, P, LNG, P, P, I, I, I, I, I, P, P, P],
            "la_moe_pairs": [I, P, P, P, P, P, P, I, I, I, I, I, P, P, I, F, F, P],
            "la_sinusoid_add": [P, I, I, P, P, P],
            "la_qk_norm_pages": [I, P, I, I, I, I, I, I, I, P, P, F, F, I, P, P, P, I, P],
            "la_mamba2": [I, P, I, I, I, I, I, I, I, I, P, P, P, P, P, P, P, I, F, P, P, P, P, P, I, P, P, P, P, P, P, I,
                          P],
            "la_attn_latent": [P, P, P, P, P, I, I, I, I, I, I, F, I, P, I, P, I, P, P, P],
            "la_norm_chain": [P, I, I, P, I, LNG, I, I, F, P, P, F, P, I, I, F, P, P, P, I, P],
            "la_add_group_norm": [P, I, I, P, I, LNG, I, P, F, I, P, I, P],
            "la_poly_norm_act": [P, I, LNG, I, I, I, P, F, P, I, P],
            "la_sigmoid_mul": [P, I, P, I, LNG, I, I, P, I, P],
            "la_qk_norm_rope_pages": [I, P, LNG, I, I, I, I, I, P, P, P, P, F, P, F, I, P, P, P, P, I, P],
            "la_rotate_heads": [I, P, I, I, I, P, P, F, F, P, LNG, P],
            "la_delta_rule": [I, P, LNG, P, P, I, I, I, I, I, I, I, I, P, P, P, P, P, F, F, P, P, P, P, P, I, P, P, P, P,
                              P, P, P],
            "la_matrix_memory": [I, P, LNG, I, I, I, I, I, P, F, P, F, F, F, P, P, P, P, P, I, P, P, P, P, P, LNG, P, I,
                                 P],
            "la_glu_clamp": [P, I, LNG, I, I, I, F, F, P, I, P],
            "la_side_gate": [P, I, LNG, I, I, I, P, P, I, I, P, I, P],
            "la_rope_pages": [I, P, I, I, I, I, I, I, P, P, P, F, I, I, I, P, P, P, I, P],
            "la_latent_kv": [I, P, I, I, I, P, F, P, P, P, F, I, P, I, P],
            "la_retention": [I, P, I, I, I, I, I, P, P, P, P, I, P, P, F, I, F, P, P, P, P, I, P],
            "la_img_resample_h": [P, I, I, P, I, P, P, I, P],
            "la_img_resample_v_tiles": [P, I, I, P, P, I, I, I, I, I, I, I, P, P, P, P, P],
        }
        missing = []
        for name, args in sig.items():
            try:
                fn = getattr(L, name)
            except AttributeError:
                # a library older than these bindings (an A/B build, a stale .so): everything else
                # still binds; calling the missing entry point fails loudly (ctypes AttributeError)
                missing.append(name)
                continue
            fn.argtypes = args
            fn.restype = I
        if missing and not partial:
            import warnings
            warnings.warn(f"{path.name} lacks {', '.join(missing)}: rebuild it (python -c 'from localai_amd.ops "
                          f"import _build; _build.build()')")
        if hasattr(L, "la_gemm_scales_bytes"):
            L.la_gemm_scales_bytes.argtypes = [I, I]
            L.la_gemm_scales_bytes.restype = LNG
        gv = os.environ.get("LOCALAI_AMD_GEMV_VARIANT")
        if gv is not None:
            _check(L.la_gemv_variant(int(gv)), "la_gemv_variant")
        mt = os.environ.get("LOCALAI_AMD_MOE_TUNE")  # "row_tile,waves" of the wide-batch MoE GEMM (A/B)
        if mt:
            a, b = (int(v) for v in mt.split(","))
            _check(L.la_moe_tune(a, b), "la_moe_tune")
        if os.environ.get("LOCALAI_AMD_DEC_ONE_PART") and hasattr(L, "la_dec_one_part"):
            _check(L.la_dec_one_part(int(os.environ["LOCALAI_AMD_DEC_ONE_PART"])), "la_dec_one_part")
        _LIB = L
        return L


def _has(name: str) -> bool:
    """Is the entry point in the loaded library (a partial library, require_kernels, lacks the GEMM
    families its model does not launch: those shapes take the library GEMM instead)."""
    return hasattr(lib(), name)


def hip_available() -> bool:
    try:
        lib()
        return True
    except Exception:
        return False


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check(rc: int, name: str):
    if rc != 0:
        raise RuntimeError(f"{name} failed with code {rc}")


# ---------------------------------------------------------------------------------------
# Quantised weights
# ---------------------------------------------------------------------------------------

@dataclass
class QWeight:
    """A [N, K] matrix in a runtime layout (see csrc/qweight.h)."""
    fmt: int
    N: int
    K: int
    planes: Tuple[Optional[torch.Tensor], ...]   # p0..p3 device planes (GPU path)
    ref: Optional[torch.Tensor] = None            # fp32 [N, K] (CPU path / oracle)
    bf16: Optional[torch.Tensor] = None           # optional HBM-resident bf16 copy (prefill GEMMs)
    gsc: Optional[torch.Tensor] = None            # blocked per-(column, K-step) scale plane (gemm_q.hip)

    @property
    def device(self) -> torch.device:
        t = self.planes[0] if self.planes and self.planes[0] is not None else self.ref
        return t.device

    @property
    def nbytes(self) -> int:
        return sum(p.numel() * p.element_size() for p in self.planes if p is not None)

    @staticmethod
    def from_raw(raw: np.ndarray, ggml_type: int, shape: Tuple[int, int], device: torch.device,
                 keep_ref: bool = False) -> "QWeight":
        """raw: uint8 GGUF payload of a [N, K] tensor."""
        N, K = int(shape[0]), int(shape[1])
        t = int(ggml_type)
        if device.type != "cuda":
            ref = torch.from_numpy(dequantize(raw, t, (N, K)).astype(np.float32))
            fmt = {GGMLType.Q4_K: FMT_Q4_K, GGMLType.Q6_K: FMT_Q6_K, GGMLType.Q8_0: FMT_Q8_0}.get(t, FMT_BF16)
            return QWeight(fmt, N, K, (None, None, None, None), ref=ref)
        ref = torch.from_numpy(dequantize(raw, t, (N, K)).astype(np.float32)) if keep_ref else None
        with warnings.catch_warnings():
            # raw is usually a read-only view of the mmapped GGUF; the host tensor is only read
            # by the device copy, so wrap it without a host-side copy of the payload
            warnings.filterwarnings("ignore", message="The given NumPy array is not writable")
            src = torch.from_numpy(np.ascontiguousarray(raw)).to(device, non_blocking=False)
        if t == GGMLType.Q4_K and K % 256 == 0:
            b = src.view(N, K // 256, 144)
            qs = b[:, :, 16:].contiguous().view(N, K // 2)
            hdr = b[:, :, :16].contiguous().view(N, K // 256 * 16)
            scm, dd = _q4k_gemv_planes(b[:, :, :16])
            return QWeight(FMT_Q4_K, N, K, (qs, hdr, scm, dd), ref=ref)
        if t == GGMLType.Q6_K and K % 256 == 0:
            b = src.view(N, K // 256, 210)
            ql = b[:, :, :128].contiguous().view(N, K // 2)
            qh = b[:, :, 128:192].contiguous().view(N, K // 4)
            sc = b[:, :, 192:208].contiguous().view(N, K // 16)
            d = b[:, :, 208:210].contiguous().view(N, K // 256 * 2)
            return QWeight(FMT_Q6_K, N, K, (ql, qh, sc, d), ref=ref)
        if t == GGMLType.Q8_0 and K % 256 == 0:
            b = src.view(N, K // 32, 34)
            d = b[:, :, :2].contiguous().view(N, K // 32 * 2)
            qs = b[:, :, 2:].contiguous().view(N, K)
            return QWeight(FMT_Q8_0, N, K, (qs, d, None, None), ref=ref)
        # anything else: materialise bf16 (dequantised on the host once)
        w = torch.from_numpy(dequantize(raw, t, (N, K)).astype(np.float32)).to(device).to(torch.bfloat16)
        return QWeight(FMT_BF16, N, K, (w.view(torch.uint8).view(N, K * 2), None, None, None), ref=ref)

    @staticmethod
    def from_float(w: torch.Tensor) -> "QWeight":
        """Dense bf16 weight (used for tensors stored as F16/F32 or built in memory)."""
        N, K = w.shape
        if w.device.type != "cuda":
            return QWeight(FMT_BF16, N, K, (None, None, None, None), ref=w.float())
        wb = w.to(torch.bfloat16).contiguous()
        return QWeight(FMT_BF16, N, K, (wb.view(torch.uint8).view(N, K * 2), None, None, None))

    @staticmethod
    def from_f32(w: torch.Tensor) -> "QWeight":
        """Dense fp32 weight for the 32-bit serving mode (linear_multi: x fp32 @ W^T by the library SGEMM)."""
        N, K = w.shape
        if w.device.type != "cuda":
            return QWeight(FMT_F32, N, K, (None, None, None, None), ref=w.float())
        wf = w.float().contiguous()
        return QWeight(FMT_F32, N, K, (wf.view(torch.uint8).view(N, K * 4), None, None, None))

    def f32(self) -> torch.Tensor:
        return self.planes[0].view(torch.float32).view(self.N, self.K)

    def ptrs(self):
        return [_ptr(p) for p in self.planes]

    @property
    def gemv_ok(self) -> bool:
        """Has the planes the int8-dot decode GEMV (gemv_dp4.hip) reads."""
        return (self.fmt == FMT_Q6_K or (self.fmt == FMT_Q4_K and self.planes[2] is not None)
                or (self.fmt == FMT_Q8_0 and self.planes[1] is not None)) and self.K % 256 == 0

    def materialize_bf16(self) -> torch.Tensor:
        """HBM-resident bf16 copy for the large-M (prefill) GEMM path."""
        if self.bf16 is None:
            if self.device.type != "cuda":
                self.bf16 = self.ref.to(torch.bfloat16)
            elif self.fmt == FMT_BF16:
                self.bf16 = self.planes[0].view(torch.bfloat16).view(self.N, self.K)
            else:
                out = torch.empty(self.N, self.K, dtype=torch.bfloat16, device=self.device)
                _check(lib().la_dequant(self.fmt, *self.ptrs(), self.N, self.K, out.data_ptr(), _stream()),
                       "la_dequant")
                self.bf16 = out
        return self.bf16

    @property
    def tile_ok(self) -> bool:
        """Can feed the quantised tile GEMM (gemm_q.hip)."""
        return self.K % 256 == 0 and self.fmt in (FMT_Q4_K, FMT_Q6_K, FMT_Q8_0, FMT_BF16) and self.planes[0] is not None

    def tile_planes(self) -> Tuple[int, Optional[int], Optional[int]]:
        """(p0, p1, gsc) pointers for la_qgemm_tile; the 8-byte-per-(column, K-step) scale plane
        is built on the device on first use (0.125 B per weight)."""
        if self.fmt == FMT_BF16:
            return _ptr(self.planes[0]), None, None
        if self.gsc is None:
            nbytes = int(lib().la_gemm_scales_bytes(self.N, self.K))
            g = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
            if self.fmt == FMT_Q4_K:
                if self.planes[2] is None:
                    raise ValueError("Q4_K weight without its unpacked scale planes")
                a, b = self.planes[2], self.planes[3]
            elif self.fmt == FMT_Q6_K:
                a, b = self.planes[2], self.planes[3]
            else:
                a, b = self.planes[1], None
            _check(lib().la_gemm_scales(self.fmt, _ptr(a), _ptr(b), self.N, self.K, g.data_ptr(), _stream()),
                   "la_gemm_scales")
            self.gsc = g
        p1 = _ptr(self.planes[1]) if self.fmt == FMT_Q6_K else None
        return _ptr(self.planes[0]), p1, self.gsc.data_ptr()

    def dequant_f32(self) -> torch.Tensor:
        if self.ref is not None:
            return self.ref
        return self.materialize_bf16().float()

    def shard(self, dim: int, rank: int, world: int) -> "QWeight":
        """Row (dim=0) or column (dim=1) shard for tensor parallelism.  Column shards
        must stay aligned to 256-wide super-blocks."""
        if world == 1:
            return self
        if dim == 0:
            n = self.N // world
            sl = slice(rank * n, (rank + 1) * n)
            planes = tuple(None if p is None else p[sl].contiguous() for p in self.planes)
            ref = None if self.ref is None else self.ref[sl].contiguous()
            return QWeight(self.fmt, n, self.K, planes, ref=ref)
        k = self.K // world
        if k % 256:
            raise ValueError(f"column shard {k} not a multiple of 256")
        ref = None if self.ref is None else self.ref[:, rank * k:(rank + 1) * k].contiguous()
        planes = []
        for p in self.planes:
            if p is None:
                planes.append(None)
                continue
            per_row = p.shape[1]
            c = per_row // world
            planes.append(p[:, rank * c:(rank + 1) * c].contiguous())
        return QWeight(self.fmt, self.N, k, tuple(planes), ref=ref)


def _q4k_gemv_planes(h: torch.Tensor):
    """From Q4_K block headers h [N, nsb, 16] (f16 d, f16 dmin, 12 packed 6-bit scales/mins)
    build the two planes the decode GEMV reads: scm [N, nsb*16] = (sc0,m0,sc1,m1,...) and
    dd [N, nsb*4] = (d, dmin).  Unpacking is ggml's get_scale_min_k4 [external, llama.cpp
    ggml-quants.c], done once at load instead of per lane per step."""
    N, nsb, _ = h.shape
    q = h[:, :, 4:16].to(torch.int32)
    sc = torch.empty(N, nsb, 8, dtype=torch.int32, device=h.device)
    mn = torch.empty_like(sc)
    sc[..., :4] = q[..., 0:4] & 63
    mn[..., :4] = q[..., 4:8] & 63
    sc[..., 4:] = (q[..., 8:12] & 0xF) | ((q[..., 0:4] >> 6) << 4)
    mn[..., 4:] = (q[..., 8:12] >> 4) | ((q[..., 4:8] >> 6) << 4)
    scm = torch.stack([sc, mn], -1).to(torch.uint8).reshape(N, nsb * 16).contiguous()
    dd = h[:, :, :4].contiguous().view(N, nsb * 4)
    return scm, dd


def concat_rows(ws: Sequence[QWeight]) -> Optional[QWeight]:
    """Fuse weights with equal format and K along N (QKV, gate|up).  None if impossible."""
    if not ws or len({(w.fmt, w.K) for w in ws}) != 1:
        return None
    w0 = ws[0]
    planes = []
    for i in range(4):
        ps = [w.planes[i] for w in ws]
        planes.append(None if ps[0] is None else torch.cat(ps, 0))
    ref = None if w0.ref is None else torch.cat([w.ref for w in ws], 0)
    return QWeight(w0.fmt, sum(w.N for w in ws), w0.K, tuple(planes), ref=ref)


def fuse_runs(ws: Sequence[QWeight]) -> List[QWeight]:
    """Concatenate each run of consecutive weights that share format and K (one GEMM launch
    per run); the output column order is unchanged."""
    out: List[QWeight] = []
    run: List[QWeight] = []
    for w in ws:
        if run and (w.fmt, w.K) != (run[0].fmt, run[0].K):
            out.append(concat_rows(run) if len(run) > 1 else run[0])
            run = []
        run.append(w)
    if run:
        out.append(concat_rows(run) if len(run) > 1 else run[0])
    return out


# ---------------------------------------------------------------------------------------
# Partial results: S fp32 split-K slabs [S, M, N] or one bf16/fp32 [M, N] matrix
# ---------------------------------------------------------------------------------------

@dataclass
class Partial:
    t: torch.Tensor              # [S, M, N] f32 or [M, N] bf16/f32
    bias: Optional[torch.Tensor] = None

    @property
    def S(self) -> int:
        return self.t.shape[0] if self.t.dim() == 3 else 0

    @property
    def M(self) -> int:
        return self.t.shape[-2]

    @property
    def N(self) -> int:
        return self.t.shape[-1]

    def src_args(self):
        if self.t.dim() == 3:
            assert self.t.dtype == torch.float32
            return (self.t.data_ptr(), self.t.shape[1] * self.t.shape[2], self.t.shape[0], _ptr(self.bias))
        assert self.t.dtype == torch.bfloat16, "single-matrix sources must be bf16"
        return (self.t.data_ptr(), 0, 0, _ptr(self.bias))

    def dense(self) -> torch.Tensor:
        x = self.t.float().sum(0) if self.t.dim() == 3 else self.t.float()
        if self.bias is not None:
            x = x + self.bias.float()
        return x

    def cols(self, a: int, b: int) -> "Partial":
        t = self.t[..., a:b].contiguous()
        bias = None if self.bias is None else self.bias[a:b]
        return Partial(t, bias)


def pick_splits(N: int, K: int, M: int) -> int:
    """Split-K so the skinny GEMM launches >= ~2 workgroups per CU (256 CUs)."""
    nsb = K // 256
    nblk = (N + 63) // 64
    want = max(1, math.ceil(512 / nblk))
    best = 1
    for s in range(1, nsb + 1):
        if nsb % s == 0:
            best = s
            if s >= want:
                break
    # the consumer reads S slabs: keep the slab traffic below the weight traffic
    while best > 1 and best * M * N * 4 * 2 > N * K // 2:
        cands = [s for s in range(1, best) if nsb % s == 0]
        best = cands[-1] if cands else 1
    return best


GEMV_MAX_SPLITS = int(os.environ.get("LOCALAI_AMD_GEMV_MAX_SPLITS", "0"))   # 0: no cap (A/B knob)


def _gemv_splits(ws, K: int, M: int) -> int:
    """Split-K for the dp4 GEMV: ~2 workgroups per CU (pick_splits), then grown until the
    workgroup's int8 activation image (kper bytes + 16-run sums + scales per row) fits 64 KiB."""
    nsb = K // 256
    S = min(pick_splits(w.N, w.K, M) for w in ws)
    if all(w.fmt == FMT_Q8_0 for w in ws):
        # 1.06 B/weight (vs 0.56 for Q4_K): each split already streams twice the bytes, and half
        # the splits measured fastest (Llama-3-8B Q8_0, M=1: o 9.7 -> 7.8 us, q|k|v 12.7 -> 9.8 us)
        S = max(1, S // 2)
    if M == 1 and K >= 24576:
        # 70B-class down projections (K = 28672): 7 splits measured 9 % faster than 4 for Q6_K and
        # 4 % for Q4_K (profiles/r3_session2_measurements.md, scripts/gemv_sweep.py --preset 70b)
        S = max(S, 7)
    if GEMV_MAX_SPLITS:
        S = min(S, GEMV_MAX_SPLITS)
    while nsb % S:
        S -= 1
    mt = 1 if M == 1 else (2 if M == 2 else 4)
    while mt * (K // S) * (1 + 4 / 16 + 4 / 32) > 65536:
        S = next(s for s in range(S + 1, nsb + 1) if nsb % s == 0)
    return S


def gemv_dp4(x: Optional[torch.Tensor], ws: Sequence[QWeight], S: int, out: torch.Tensor,
             act_src: Optional[Partial] = None, act_mode: int = 0) -> None:
    """out[S, M, sum(N)] = split-K partials of x @ [W0; W1; ...]^T from the int8-dot decode GEMV,
    up to 3 weights (mixed Q4_K / Q6_K, same K) per launch.  With act_src (fp32 gate|up slabs)
    x = act(act_src) is formed inside the GEMV prologue instead of being read."""
    M = out.shape[1]
    K = ws[0].K
    a = (None, 0, 0, None) if act_src is None else act_src.src_args()
    Ntot = out.shape[-1]
    # launch groups: <= 3 weights whose formats form at most two runs [FA ...][FB ...]
    groups: List[List[QWeight]] = []
    for w in ws:
        g = groups[-1] if groups else None
        if (g is not None and len(g) < 3 and (len({v.fmt for v in g}) == 1 or w.fmt == g[-1].fmt)
                and (w.fmt == FMT_Q8_0) == (g[0].fmt == FMT_Q8_0)):  # Q8_0 launches are homogeneous
            g.append(w)
        else:
            groups.append([w])
    col = 0
    for seg in groups:
        n = len(seg)
        fmts = (ctypes.c_int * n)(*[w.fmt for w in seg])
        planes = (ctypes.c_void_p * (4 * n))(*[p for w in seg for p in w.ptrs()])
        Ns = (ctypes.c_int * n)(*[w.N for w in seg])
        args = (n, fmts, planes, Ns, K, None if x is None else x.data_ptr(), K, M, S, out.data_ptr() + col * 4,
                Ntot, M * Ntot, a[0], a[1], a[2], a[3], act_mode)
        _check(lib().la_qgemv_dp4(*args, _stream()), "la_qgemv_dp4")
        col += sum(w.N for w in seg)


# off by default: measured neutral on Llama-3-8B C=1 (profiles/r4_c1_fused_norm.md) -- the 33
# add_norm launches go away, but every q|k|v workgroup re-reads the residual plus the down
# projection's 8 split-K slabs (144 KiB from L2 per workgroup) and the GEMV grows by the same ~4 us
GEMV_NORM = os.environ.get("LOCALAI_AMD_GEMV_NORM", "0") == "1"


@dataclass
class NormIn:
    """A deferred layer-boundary residual-add + RMSNorm, handed to the consuming decode GEMV
    instead of a materialised bf16 x: x = rmsnorm(res + add) * weight is formed in the GEMV
    prologue (gemv_dp4.hip GV_NORM) and the updated residual lands in res_out (written once, by
    one workgroup; None when there is no add).  Removes the add_norm launch at every layer
    boundary of a batch-1/2 decode step (SURVEY §2.8 K2 + K14 folded into K5)."""
    res: torch.Tensor               # fp32 [M, D]
    add: Optional[Partial]          # fp32 split-K slabs [S, M, D] or None
    weight: torch.Tensor            # fp32 [D]
    eps: float
    res_out: Optional[torch.Tensor]  # fp32 [M, D], not res; None iff add is None

    @property
    def shape(self):
        return self.res.shape

    @property
    def is_cuda(self) -> bool:
        return self.res.is_cuda

    def args(self):
        a = self.add.src_args() if self.add is not None else (None, 0, 0, None)
        return (self.res.data_ptr(), a[0], a[1], a[2], a[3], self.weight.data_ptr(), float(self.eps),
                _ptr(self.res_out))

    def materialize(self) -> torch.Tensor:
        """The same x through add_norm (residual updated in res, then copied to res_out)."""
        xn = add_norm(self.res, self.add, self.weight, None, self.eps, 0)
        if self.res_out is not None:
            self.res_out.copy_(self.res)
        return xn


def norm_in_ok(res: torch.Tensor, add: Optional[Partial], weight: torch.Tensor, bias) -> bool:
    """A NormIn can feed the fused GEMV prologue: GPU, fp32 residual of <= GEMV_MAX_M rows and
    width <= 8192, fp32 weight, no norm bias (RMSNorm), the add as fp32 split-K slabs."""
    M, D = res.shape
    return (GEMV_NORM and GEMV_DP4 and res.is_cuda and res.dtype == torch.float32 and M <= GEMV_MAX_M
            and D <= 8192 and D % 256 == 0 and bias is None and weight.dtype == torch.float32
            and (add is None or (add.t.dim() == 3 and add.t.dtype == torch.float32 and add.S <= 16
                                 and add.N == D)))


def qkv_rope_ok(x: torch.Tensor, ws: Sequence[QWeight], bias, mode: int, rot: int, Dh: int, block_size: int) -> bool:
    """The fused decode q|k|v GEMV + RoPE + KV append (gemv_dp4.hip GVRope) applies: GPU, batch
    <= GEMV_MAX_M, Q4_K/Q6_K weights, no bias, NORM rotary over the whole head."""
    return (x.is_cuda and GEMV_DP4 and x.shape[0] <= GEMV_MAX_M and bias is None and mode == 0 and rot == Dh
            and Dh % 2 == 0 and block_size % 8 == 0 and len(ws) <= 3 and all(w.gemv_ok for w in ws)
            and len({w.K for w in ws}) == 1 and ws[0].K % 1024 == 0
            and len({w.fmt == FMT_Q8_0 for w in ws}) == 1)


def qkv_rope_dp4(x: torch.Tensor, ws: Sequence[QWeight], pos: torch.Tensor, slots: torch.Tensor,
                 cos_sin: torch.Tensor, Hq: int, Hkv: int, Dh: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 block_size: int, q_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q = rope(x @ Wq^T) [M, Hq, Dh] bf16; k = rope(x @ Wk^T) and v = x @ Wv^T appended to the paged
    cache at `slots` -- one GEMV launch (split-K 1) with the rotation and the append in its
    epilogue, instead of a GEMV + rope_kv."""
    M, K = x.shape
    if isinstance(x, NormIn):
        if q_out is None:
            q_out = torch.empty(M, Hq, Dh, dtype=torch.bfloat16, device=x.res.device)
        if sum(w.N for w in ws) != (Hq + 2 * Hkv) * Dh:
            raise ValueError("qkv_rope_dp4: weights do not form q|k|v")
        n = len(ws)
        fmts = (ctypes.c_int * n)(*[w.fmt for w in ws])
        planes = (ctypes.c_void_p * (4 * n))(*[p for w in ws for p in w.ptrs()])
        Ns = (ctypes.c_int * n)(*[w.N for w in ws])
        _check(lib().la_qgemv_dp4_rope_norm(n, fmts, planes, Ns, K, M, pos.data_ptr(), slots.data_ptr(),
                                            cos_sin.data_ptr(), Hq, Hkv, Dh, q_out.data_ptr(), k_cache.data_ptr(),
                                            v_cache.data_ptr(), block_size, *x.args(), _stream()),
               "la_qgemv_dp4_rope_norm")
        return q_out
    if x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("qkv_rope_dp4: x must be contiguous bf16")
    if sum(w.N for w in ws) != (Hq + 2 * Hkv) * Dh:
        raise ValueError("qkv_rope_dp4: weights do not form q|k|v")
    if pos.dtype != torch.int32 or slots.dtype != torch.int32 or pos.numel() < M or slots.numel() < M:
        raise ValueError("qkv_rope_dp4: pos / slots must be int32 [M]")
    if q_out is None:
        q_out = torch.empty(M, Hq, Dh, dtype=torch.bfloat16, device=x.device)
    n = len(ws)
    fmts = (ctypes.c_int * n)(*[w.fmt for w in ws])
    planes = (ctypes.c_void_p * (4 * n))(*[p for w in ws for p in w.ptrs()])
    Ns = (ctypes.c_int * n)(*[w.N for w in ws])
    _check(lib().la_qgemv_dp4_rope(n, fmts, planes, Ns, K, x.data_ptr(), M, pos.data_ptr(), slots.data_ptr(),
                                   cos_sin.data_ptr(), Hq, Hkv, Dh, q_out.data_ptr(), k_cache.data_ptr(),
                                   v_cache.data_ptr(), block_size, _stream()), "la_qgemv_dp4_rope")
    return q_out


SKINNY_MAX_M = 64
GEMV_MAX_M = 2           # M <= GEMV_MAX_M: int8-dot decode GEMV (gemv_dp4.hip, supports M <= 4) on Q4_K/Q6_K
GEMV_DP4 = os.environ.get("LOCALAI_AMD_GEMV", "dp4") == "dp4"
MID_MAX_M = 256          # 64 < M <= MID_MAX_M: quantised MFMA tile GEMMs (gemm_q.hip / gemm_q32.hip), autotuned
GEMM_AUTOTUNE = True
# (M, K, ((fmt, N), ...)) -> (kind, S, variant); filled by _autotune_mid at warm-up (eager runs
# before each decode-graph capture), consulted during capture / replay.
_GEMM_CHOICE: dict = {}


def blas_tuning_start(path: Optional[str] = None) -> bool:
    """Per-shape solution search for the library (hipBLASLt / rocBLAS) GEMMs, run while the engine
    warms up its decode graphs: PyTorch-ROCm TunableOp times every candidate kernel of each new
    (M, N, K) against a rotating 512 MiB buffer set (cold weights, as in decode) and keeps the
    fastest.  Results persist in a CSV so a restart reuses them.  Tuning is switched off again
    before serving (blas_tuning_stop): prefill chunk sizes vary and must never tune inline."""
    if os.environ.get("LOCALAI_AMD_BLAS_TUNE", "1") == "0" or not torch.cuda.is_available():
        return False
    try:
        import torch.cuda.tunable as tn
    except ImportError:
        return False
    if path is None:
        root = os.environ.get("LOCALAI_AMD_CACHE") or os.path.join(os.path.expanduser("~"), ".cache", "localai_amd")
        os.makedirs(root, exist_ok=True)
        dev = torch.cuda.current_device()
        name = torch.cuda.get_device_properties(dev).gcnArchName.split(":")[0]
        # one file per device: data-parallel ranks on one node tune (and write) concurrently
        path = os.path.join(root, f"tunableop_{name}_dev{dev}.csv")
    tn.enable(True)
    tn.set_filename(path)
    if os.path.exists(path):
        try:
            tn.read_file(path)
        except Exception:  # noqa: BLE001 - a stale/corrupt cache only costs a re-tune
            pass
    tn.set_max_tuning_duration(int(os.environ.get("LOCALAI_AMD_BLAS_TUNE_MS", "15")))
    tn.set_max_tuning_iterations(20)
    try:
        tn.set_rotating_buffer_size(512)
    except Exception:  # noqa: BLE001
        pass
    tn.tuning_enable(True)
    return True


class blas_tuning_paused:
    """Context: library GEMMs inside run on already-tuned or default solutions without tuning new
    shapes.  For GEMMs whose M changes every step (a MoE expert's routed rows during prefill): each
    new (M, N, K) would otherwise be tuned during warm-up -- hundreds of shapes, minutes of start-up."""

    def __enter__(self):
        self.prev = False
        if not torch.cuda.is_available():
            return self
        try:
            import torch.cuda.tunable as tn
            self.prev = tn.is_enabled() and tn.tuning_is_enabled()
            if self.prev:
                tn.tuning_enable(False)
        except (ImportError, RuntimeError):
            pass
        return self

    def __exit__(self, *exc):
        if self.prev:
            import torch.cuda.tunable as tn
            tn.tuning_enable(True)
        return False


def blas_tuning_stop() -> None:
    import torch.cuda.tunable as tn
    tn.tuning_enable(False)   # keep using the tuned solutions, never tune inline while serving
    try:
        tn.write_file()
    except Exception:  # noqa: BLE001
        pass


def fuse_bf16(ws: Sequence[QWeight]) -> Optional[torch.Tensor]:
    """One HBM-resident bf16 [sum(N), K] matrix behind several weights that feed one output
    (a Q4_K q|k with a Q6_K v): each weight's bf16 copy becomes a row slice of it, so the
    library path runs ONE GEMM for the fused output instead of one per format (at decode
    batch 256 the separate v GEMM cost a launch of its own: 12.5 us x 16 layers per step).
    No extra memory: the per-weight copies are the slices."""
    if len(ws) < 2 or any(w.device.type != "cuda" or w.K != ws[0].K for w in ws):
        return None
    base = getattr(ws[0], "_fused_bf16", None)
    if base is not None and base.shape[0] == sum(w.N for w in ws):
        return base
    Ntot, K = sum(w.N for w in ws), ws[0].K
    fused = torch.empty(Ntot, K, dtype=torch.bfloat16, device=ws[0].device)
    row = 0
    for w in ws:
        fused[row:row + w.N].copy_(w.materialize_bf16())
        w.bf16 = fused[row:row + w.N]
        row += w.N
    ws[0]._fused_bf16 = fused
    return fused


_SCRATCH: dict = {}
_SCRATCH_LOCK = threading.Lock()


def _scratch(device, need: int) -> torch.Tensor:
    """bf16 dequant scratch of >= need elements for the calling thread.

    One buffer per (device, thread): two engines serving from different threads on one GPU
    (in-process whisper / CLIP / a second LLM) enqueue their dequant + GEMM pairs interleaved,
    so a shared buffer would hand one engine's GEMM the other's weights.  Entries of threads that
    have exited are dropped on the next call, so an executor pool's turnover does not keep one
    large buffer per dead thread (VRAM outside the KV budget).  Inside a stream capture the buffer
    is allocated fresh from the graph's private pool instead: a replayed graph must never write
    into memory that a later (larger) scratch reallocation returned to the caching allocator."""
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(need, dtype=torch.bfloat16, device=device)
    key = (device, threading.get_ident())
    with _SCRATCH_LOCK:
        buf = _SCRATCH.get(key)
        if buf is None or buf.numel() < need:
            live = {t.ident for t in threading.enumerate()}
            for k in [k for k in _SCRATCH if k[1] not in live]:
                del _SCRATCH[k]
            _SCRATCH.pop(key, None)
            buf = _SCRATCH[key] = torch.empty(need, dtype=torch.bfloat16, device=device)
    return buf


def release_scratch(device=None) -> None:
    """Drop the calling thread's dequant scratch (a non-engine caller after a large GEMM)."""
    with _SCRATCH_LOCK:
        for k in [k for k in _SCRATCH if k[1] == threading.get_ident() and (device is None or k[0] == device)]:
            del _SCRATCH[k]


def _run_scratch_blas(x, ws, Ntot):
    """Large-M (prefill chunk) GEMM: dequantise the weights into a per-thread bf16 scratch
    buffer (reused by every call, sized by the largest fused weight seen), then a library GEMM
    on it -- the reference's own large-batch path (ggml convert.cu dequant + hipBLAS GemmEx,
    SURVEY K7), without a persistent bf16 copy of the model.  The dequant streams the quantised
    bytes once and writes 2 B/weight: ~6 % of a 8192-row chunk's GEMM time.  A lone bf16 weight
    is multiplied in place (no copy)."""
    K = x.shape[1]
    if len(ws) == 1 and ws[0].fmt == FMT_BF16:
        return torch.matmul(x, ws[0].planes[0].view(torch.bfloat16).view(ws[0].N, K).t())
    need = Ntot * K
    wt = _scratch(x.device, need)[:need].view(Ntot, K)
    row = 0
    for w in ws:
        if w.fmt == FMT_BF16:
            wt[row:row + w.N].copy_(w.planes[0].view(torch.bfloat16).view(w.N, w.K))
        else:
            _check(lib().la_dequant(w.fmt, *w.ptrs(), w.N, w.K, wt[row:row + w.N].data_ptr(), _stream()), "la_dequant")
        row += w.N
    return torch.matmul(x, wt.t())


def _run_blas(x, ws, Ntot):
    if TILE_GEMM and all(w.bf16 is None for w in ws) and getattr(ws[0], "_fused_bf16", None) is None:
        return _run_scratch_blas(x, ws, Ntot)
    if len(ws) == 1:
        return torch.matmul(x, ws[0].materialize_bf16().t())
    fused = getattr(ws[0], "_fused_bf16", None)
    if fused is not None and fused.shape[0] == Ntot:
        return torch.matmul(x, fused.t())
    y = torch.empty(x.shape[0], Ntot, dtype=torch.bfloat16, device=x.device)
    col = 0
    for w in ws:
        torch.matmul(x, w.materialize_bf16().t(), out=y[:, col:col + w.N])
        col += w.N
    return y


_FLUSH: dict = {}


def _cold_caches(device):
    """Evict L2 and the 256 MiB Infinity Cache by READING a 384 MiB scratch buffer (a write
    flush leaves dirty lines whose write-back then taxes the timed call), so a timed GEMM
    reads its weights from HBM as it does in the engine, where every decode step streams the
    whole model once."""
    buf = _FLUSH.get(device)
    if buf is None:
        buf = _FLUSH[device] = torch.ones(96 << 20, dtype=torch.float32, device=device)
    buf.sum()


# Quantised tile GEMM (gemm_q.hip): the M > SKINNY_MAX_M path.  Tile ids: (BM, BN).
GQ_TILES = {0: (256, 256), 1: (256, 128), 2: (128, 256), 3: (128, 128), 4: (256, 64), 5: (64, 256), 6: (256, 256),
            7: (128, 256), 8: (256, 128), 12: (128, 128), 14: (64, 256),
            # software-pipelined schedules of 0, 1, 3, 6, 7
            10: (256, 256), 11: (256, 128), 13: (128, 128), 16: (256, 256), 17: (128, 256)}
# LOCALAI_AMD_TILE_GEMM=0 restores the round-2 path (hipBLASLt on bf16 weight copies)
TILE_GEMM = os.environ.get("LOCALAI_AMD_TILE_GEMM", "1") == "1"
# M > MID_MAX_M (prefill chunks): "blas" = dequantise into a scratch buffer + library GEMM, "tile" =
# gemm_q.hip.  "blas" stays the default: the in-kernel-dequant MFMA GEMMs (gemm_bs.hip, and round
# 5's gemm_pp.hip before it) top out near 1.0 PF/s against hipBLASLt's 1.3 at M = 8192
# (profiles/r6_gemm_bs.md, r5_prefill_gemm.md)
PREFILL_GEMM = os.environ.get("LOCALAI_AMD_PREFILL_GEMM", "blas")


def _tile_split_ok(K: int, S: int) -> bool:
    ks = K // 64
    return S >= 1 and -(-ks // S) * (S - 1) < ks


_TILE2_PAIRS = {(FMT_Q4_K, FMT_Q6_K), (FMT_Q6_K, FMT_Q4_K)}
_TILE2_TILES = (7, 8, 12)


def _run_tile(x, ws, S, out, Ntot, tile):
    """out: fp32 slabs [S, M, Ntot], or a bf16 [M, Ntot] matrix (S == 1).  Two weights of a
    Q4_K/Q6_K mix (q|k + v) run as ONE launch (la_qgemm_tile2)."""
    M, K = x.shape
    bf = out.dtype == torch.bfloat16
    esz = 2 if bf else 4
    if len(ws) == 2 and (ws[0].fmt, ws[1].fmt) in _TILE2_PAIRS and tile in _TILE2_TILES:
        a0, a1, ag = ws[0].tile_planes()
        b0, b1, bg = ws[1].tile_planes()
        _check(lib().la_qgemm_tile2(ws[0].fmt, a0, a1, ag, ws[0].N, ws[1].fmt, b0, b1, bg, ws[1].N, K, x.data_ptr(), K,
                                    M, S, out.data_ptr(), Ntot, 0 if bf else M * Ntot, int(bf), tile, _stream()),
               "la_qgemm_tile2")
        return
    col = 0
    for w in ws:
        p0, p1, g = w.tile_planes()
        _check(lib().la_qgemm_tile(w.fmt, p0, p1, g, w.N, w.K, x.data_ptr(), K, M, S, out.data_ptr() + col * esz,
                                   Ntot, 0 if bf else M * Ntot, int(bf), tile, 0, _stream()), "la_qgemm_tile")
        col += w.N


# 32x32x16 quantised GEMM (gemm_q32.hip): variant id -> (BM, BN).  Variants 2 / 6 (256 x 256
# tiles) are built for Q4_K only and not for two-weight launches.
Q32_TILES = {0: (256, 128), 1: (128, 256), 2: (256, 256), 3: (128, 128), 4: (256, 128), 5: (128, 256),
             6: (256, 256), 7: (128, 128), 8: (128, 256), 9: (128, 256)}
Q32_FMTS = (FMT_Q4_K, FMT_Q6_K, FMT_Q8_0)
Q32 = os.environ.get("LOCALAI_AMD_Q32", "1") == "1"


def q32_ok(ws: Sequence[QWeight], var: int) -> bool:
    """Can the 32x32x16 kernel run these weights (one launch per weight, or one for a Q4_K/Q6_K
    pair) in this variant."""
    if not Q32 or not all(w.fmt in Q32_FMTS and w.K % 256 == 0 and w.planes[0] is not None for w in ws):
        return False
    if var in (2, 6):
        return all(w.fmt == FMT_Q4_K for w in ws) and len(ws) == 1
    return True


def _run_q32(x, ws, S, out, Ntot, var):
    """out: fp32 slabs [S, M, Ntot], or a bf16 [M, Ntot] matrix (S == 1).  A Q4_K/Q6_K pair (q|k +
    v) runs as ONE launch (la_qgemm32_2)."""
    M, K = x.shape
    bf = out.dtype == torch.bfloat16
    esz = 2 if bf else 4
    if len(ws) == 2 and (ws[0].fmt, ws[1].fmt) in _TILE2_PAIRS:
        a0, a1, ag = ws[0].tile_planes()
        b0, b1, bg = ws[1].tile_planes()
        _check(lib().la_qgemm32_2(ws[0].fmt, a0, a1, ag, ws[0].N, ws[1].fmt, b0, b1, bg, ws[1].N, K, x.data_ptr(), K,
                                  M, S, out.data_ptr(), Ntot, 0 if bf else M * Ntot, int(bf), var, _stream()),
               "la_qgemm32_2")
        return
    col = 0
    for w in ws:
        p0, p1, g = w.tile_planes()
        _check(lib().la_qgemm32(w.fmt, p0, p1, g, w.N, w.K, x.data_ptr(), K, M, S, out.data_ptr() + col * esz, Ntot,
                                0 if bf else M * Ntot, int(bf), var, _stream()), "la_qgemm32")
        col += w.N


# Shared-dequant-image GEMM (gemm_bs.hip): variant id -> (BM, BN).  Each weight column is
# dequantised once per workgroup into an LDS image all four waves read; X arrives by full-line
# loads through a private per-wave LDS transpose.  Decode batches (M 65..256) and prefill chunks.
BS_TILES = {0: (256, 128), 1: (128, 128), 2: (256, 256), 3: (256, 128)}
BS_FMTS = (FMT_Q4_K, FMT_Q6_K, FMT_Q8_0, FMT_BF16)
BS = os.environ.get("LOCALAI_AMD_BS", "1") == "1"


def bs_ok(ws: Sequence[QWeight]) -> bool:
    """Can gemm_bs.hip run these weights (one launch per weight, or one for a Q4_K/Q6_K pair)."""
    return BS and all(w.fmt in BS_FMTS and w.K % 256 == 0 and w.N % 4 == 0 and w.planes[0] is not None
                      for w in ws)


def _bs_grid(M: int, N: int, var: int) -> int:
    bm, bn = BS_TILES[var]
    return -(-M // bm) * -(-N // bn)


def _run_bs(x, ws, S, out, Ntot, var):
    """out: fp32 slabs [S, M, Ntot], or a bf16 [M, Ntot] matrix (S == 1).  A Q4_K/Q6_K pair (q|k +
    v) runs as ONE launch (la_bsgemm2)."""
    M, K = x.shape
    bf = out.dtype == torch.bfloat16
    esz = 2 if bf else 4
    slab = 0 if bf else M * Ntot
    if len(ws) == 2 and (ws[0].fmt, ws[1].fmt) in _TILE2_PAIRS:
        a0, a1, ag = ws[0].tile_planes()
        b0, b1, bg = ws[1].tile_planes()
        _check(lib().la_bsgemm2(ws[0].fmt, a0, a1, ag, ws[0].N, ws[1].fmt, b0, b1, bg, ws[1].N, K, x.data_ptr(), K,
                                M, S, out.data_ptr(), Ntot, slab, int(bf), var, _stream()), "la_bsgemm2")
        return
    col = 0
    for w in ws:
        p0, p1, g = w.tile_planes()
        _check(lib().la_bsgemm(w.fmt, p0, p1, g, w.N, w.K, x.data_ptr(), K, M, S, out.data_ptr() + col * esz, Ntot,
                               slab, int(bf), var, _stream()), "la_bsgemm")
        col += w.N


def _run_bs_glu(x, pair, F: int, mode: int, var: int, out) -> None:
    M, K = x.shape
    wa, oa, wb, ob = pair
    a0, a1, ag = wa.tile_planes()
    b0, b1, bg = wb.tile_planes()
    _check(lib().la_bsgemm_glu(wa.fmt, a0, a1, ag, oa, b0, b1, bg, ob, F, K, x.data_ptr(), K, M, out.data_ptr(), F,
                               mode, var, _stream()), "la_bsgemm_glu")


def _q32_grid(M: int, N: int, var: int) -> int:
    bm, bn = Q32_TILES[var]
    return -(-M // bm) * -(-N // bn)


def _tile_grid(M: int, N: int, tile: int) -> int:
    bm, bn = GQ_TILES[tile]
    return -(-M // bm) * -(-N // bn)


def pick_tile(M: int, Ns: Sequence[int], K: int) -> Tuple[int, int]:
    """Heuristic (tile, split-K) for shapes the autotuner has not seen (prefill chunks): the
    largest tile that still gives >= ~192 workgroups, else split K up to ~256 workgroups with
    every split >= 8 K-steps."""
    N = max(Ns)
    ks = K // 64
    for tile in ((6, 1, 3) if M > 128 else (7, 3, 5)):
        tiles = _tile_grid(M, N, tile)
        if tiles >= 192:
            return tile, 1
    tile = 1 if M > 128 else 3
    tiles = _tile_grid(M, N, tile)
    S = max(1, min(ks // 8, round(256 / tiles)))
    while S > 1 and not _tile_split_ok(K, S):
        S -= 1
    return tile, S


def _autotune_mid(x, ws, key, Ntot):
    """Time the tile GEMM's (tile, split-K) candidates with COLD weights (caches flushed before
    every timed call, as in decode where each step streams the whole model once) and remember
    the winner.  A split variant is charged for the extra fp32 bytes its consumer reads (at
    ~4 TB/s)."""
    M, K = x.shape
    N = max(w.N for w in ws)
    cands = []
    if all(w.tile_ok for w in ws):
        tiles = (6, 1, 7, 8, 12) if M > 128 else (7, 12, 14, 3)
        for t in tiles if _has("la_qgemm_tile") else ():
            g = _tile_grid(M, N, t)
            base = max(1, round(256 / g))
            # split-K <= 8: every split costs its consumer another fp32 [M, N] slab read
            for S in sorted({1, max(1, base // 2), base, base * 2}):
                if S <= min(8, K // 256) and _tile_split_ok(K, S):
                    cands.append(("tile", S, t))
        for v in ((9, 8, 4, 6, 0) if M > 128 else (9, 8, 7, 3)):
            if not q32_ok(ws, v) or not _has("la_qgemm32"):
                continue
            base = max(1, round(256 / _q32_grid(M, N, v)))
            for S in sorted({1, max(1, base // 2), base, base * 2}):
                if S <= min(8, K // 256) and _tile_split_ok(K, S):
                    cands.append(("q32", S, v))
    if bs_ok(ws) and _has("la_bsgemm") and (len(ws) == 1 or (len(ws) == 2 and (ws[0].fmt, ws[1].fmt) in _TILE2_PAIRS)):
        for v in ((0, 1, 3) if M > 128 else (1,)):
            base = max(1, round(256 / _bs_grid(M, N, v)))
            for S in sorted({1, max(1, base // 2), base, base * 2}):
                if S <= min(8, K // 256) and _tile_split_ok(K, S):
                    cands.append(("bs", S, v))
    if not cands or not TILE_GEMM:
        cands = [("blas", 0, 0)]
    outs = {S: torch.empty(S, M, Ntot, dtype=torch.float32, device=x.device) for _, S, _ in cands if S > 1}
    outs[1] = torch.empty(M, Ntot, dtype=torch.bfloat16, device=x.device)   # S = 1: one bf16 matrix
    best, best_t = cands[0], float("inf")
    for kind, S, t in cands:
        if kind == "blas":
            fn = lambda: _run_blas(x, ws, Ntot)  # noqa: E731
        elif kind == "tile":
            fn = lambda S=S, t=t: _run_tile(x, ws, S, outs[S], Ntot, t)  # noqa: E731
        elif kind == "bs":
            fn = lambda S=S, t=t: _run_bs(x, ws, S, outs[S], Ntot, t)  # noqa: E731
        else:
            fn = lambda S=S, t=t: _run_q32(x, ws, S, outs[S], Ntot, t)  # noqa: E731
        fn()
        ts = []
        for _ in range(3):
            _cold_caches(x.device)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) * 1000)
        tt = sorted(ts)[1]
        if kind != "blas" and S > 1:
            # fp32 slabs: written here and read back by the consumer (vs one bf16 matrix), ~4 TB/s each way
            tt += 2 * (S * M * Ntot * 4 - M * Ntot * 2) / 4e6
        if tt < best_t:
            best, best_t = (kind, S, t), tt
    _GEMM_CHOICE[key] = best
    return best


def linear(x: torch.Tensor, w: QWeight, bias: Optional[torch.Tensor] = None,
           out_slabs: Optional[torch.Tensor] = None, force: Optional[str] = None) -> Partial:
    """y = x @ W^T.  x: [M, K] bf16.  GPU: M <= 2 -> int8-dot GEMV, M <= 64 -> skinny MFMA
    kernel, larger M -> the quantised tile GEMM (gemm_q.hip); all on the quantised weights."""
    return linear_multi(x, [w], bias, out_slabs, force)


def linear_multi(x: torch.Tensor, ws: Sequence[QWeight], bias: Optional[torch.Tensor] = None,
                 out_slabs: Optional[torch.Tensor] = None, force: Optional[str] = None) -> Partial:
    """y = x @ [W0; W1; ...]^T written side by side into ONE partial (e.g. Q4_K q|k with a
    Q6_K v), so the consumer sees a single fused QKV / gate|up output."""
    M, K = x.shape
    for w in ws:
        if K != w.K:
            raise ValueError(f"linear: x has K={K}, weight has K={w.K}")
    Ntot = sum(w.N for w in ws)
    if not x.is_cuda:
        y = torch.cat([x.float() @ w.dequant_f32().t() for w in ws], -1)
        return Partial(y.to(torch.bfloat16) if force == "bf16" else y.unsqueeze(0), bias)
    if x.dtype == torch.float32 and all(w.fmt == FMT_F32 for w in ws):
        # 32-bit serving mode: the library SGEMM (torch keeps TF32-style modes off unless asked)
        y = torch.matmul(x, ws[0].f32().t()) if len(ws) == 1 else torch.cat([torch.matmul(x, w.f32().t()) for w in ws], -1)
        return Partial(y.unsqueeze(0), bias)
    if x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("linear: x must be contiguous bf16")
    if any(w.fmt == FMT_F32 for w in ws):
        raise ValueError("linear: fp32 weights take fp32 activations")
    skinny_ok = all(w.K % 256 == 0 for w in ws) and _has("la_qgemm_skinny")
    use_skinny = (M <= SKINNY_MAX_M and skinny_ok) if force is None else force == "skinny"
    tile_ok = TILE_GEMM and all(w.tile_ok for w in ws) and (_has("la_qgemm_tile") or _has("la_qgemm32") or _has("la_bsgemm"))
    S, tile, kind = 0, 0, None
    if force is not None and (force.startswith("q32:") or force.startswith("bs:")):
        kind, v, s_ = force.split(":")
        tile, S = int(v), int(s_)
    elif force is not None and force.startswith("tile"):
        # "tile" (heuristic) or "tile:<id>:<S>"
        parts = force.split(":")
        tile, S = (int(parts[1]), int(parts[2])) if len(parts) == 3 else pick_tile(M, [w.N for w in ws], K)
        kind = "tile"
    elif force is None and not use_skinny and M <= MID_MAX_M and tile_ok:
        # one tuned choice per 32-row bucket: prefill chunk / decode batch sizes vary per step
        # and must not re-run the (cache-flushing) autotune inside the serving loop
        key = ((M + 31) // 32 * 32, K, tuple((w.fmt, w.N) for w in ws))
        choice = _GEMM_CHOICE.get(key)
        if choice is None and GEMM_AUTOTUNE and not torch.cuda.is_current_stream_capturing():
            choice = _autotune_mid(x, ws, key, Ntot)
        if choice is None and tile_ok and _has("la_qgemm_tile"):
            t, s_ = pick_tile(M, [w.N for w in ws], K)
            choice = ("tile", s_, t)
        if choice is not None and choice[0] in ("tile", "q32", "bs"):
            kind, S, tile = choice
    elif force is None and not use_skinny and tile_ok and PREFILL_GEMM == "tile":
        tile, S = pick_tile(M, [w.N for w in ws], K)   # prefill: heuristic, never tuned inline
        kind = "tile"
    if kind in ("tile", "q32", "bs") and S == 1 and out_slabs is None:
        y = torch.empty(M, Ntot, dtype=torch.bfloat16, device=x.device)
        {"tile": _run_tile, "q32": _run_q32, "bs": _run_bs}[kind](x, ws, 1, y, Ntot, tile)
        return Partial(y, bias)
    if S:
        out = out_slabs
        if out is None or out.shape != (S, M, Ntot):
            out = torch.empty(S, M, Ntot, dtype=torch.float32, device=x.device)
        if kind == "tile":
            _run_tile(x, ws, S, out, Ntot, tile)
        elif kind == "bs":
            _run_bs(x, ws, S, out, Ntot, tile)
        else:
            _run_q32(x, ws, S, out, Ntot, tile)
        return Partial(out, bias)
    use_gemv = (force == "dp4") or (force is None and use_skinny and GEMV_DP4 and M <= GEMV_MAX_M
                                    and all(w.gemv_ok for w in ws))
    if use_gemv:
        if M > 4 or not all(w.gemv_ok for w in ws):
            raise ValueError("linear: dp4 GEMV needs M <= 4 and Q4_K/Q6_K weights")
        S = _gemv_splits(ws, K, M)
        out = out_slabs
        if out is None or out.shape != (S, M, Ntot):
            out = torch.empty(S, M, Ntot, dtype=torch.float32, device=x.device)
        gemv_dp4(x, ws, S, out)
        return Partial(out, bias)
    if use_skinny:
        S = min(pick_splits(w.N, w.K, M) for w in ws)
        nsb = K // 256
        while nsb % S:
            S -= 1
        out = out_slabs
        if out is None or out.shape != (S, M, Ntot):
            out = torch.empty(S, M, Ntot, dtype=torch.float32, device=x.device)
        col = 0
        for w in ws:
            dst = out.data_ptr() + col * 4
            _check(lib().la_qgemm_skinny(w.fmt, *w.ptrs(), w.N, w.K, x.data_ptr(), K, M, S, dst, Ntot,
                                         M * Ntot, _stream()), "la_qgemm_skinny")
            col += w.N
        return Partial(out, bias)
    return Partial(_run_blas(x, ws, Ntot), bias)


GLU_FUSE = os.environ.get("LOCALAI_AMD_GLU_FUSE", "1") == "1"
_GLU_CHOICE: Dict[tuple, Optional[int]] = {}


def _glu_pair(ws: Sequence[QWeight], F: int):
    """(gate weight, row offset, up weight, row offset) of a gate|up projection, or None."""
    if not all(w.tile_ok for w in ws):
        return None
    if len(ws) == 2 and ws[0].N == F and ws[1].N == F and ws[0].fmt == ws[1].fmt:
        return ws[0], 0, ws[1], 0
    if len(ws) == 1 and ws[0].N == 2 * F and F % 16 == 0:
        return ws[0], 0, ws[0], F
    return None


def _run_glu(x: torch.Tensor, pair, F: int, mode: int, tile: int, out: torch.Tensor) -> None:
    """tile < 100: gemm_q.hip tile id; 100 + v: gemm_q32.hip variant v; 200 + v: gemm_bs.hip variant v."""
    M, K = x.shape
    wa, oa, wb, ob = pair
    if tile >= 200:
        _run_bs_glu(x, pair, F, mode, tile - 200, out)
        return
    a0, a1, ag = wa.tile_planes()
    b0, b1, bg = wb.tile_planes()
    if tile >= 100:
        _check(lib().la_qgemm32_glu(wa.fmt, a0, a1, ag, oa, b0, b1, bg, ob, F, K, x.data_ptr(), K, M, out.data_ptr(),
                                    F, mode, tile - 100, _stream()), "la_qgemm32_glu")
        return
    _check(lib().la_qgemm_glu(wa.fmt, a0, a1, ag, oa, b0, b1, bg, ob, F, K, x.data_ptr(), K, M, out.data_ptr(), F,
                              mode, tile, _stream()), "la_qgemm_glu")


def _time_cold(fn) -> float:
    fn()
    ts = []
    for _ in range(3):
        _cold_caches(torch.device("cuda", torch.cuda.current_device()))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        ts.append(e0.elapsed_time(e1) * 1000)
    return sorted(ts)[1]


def glu_linear(x: torch.Tensor, ws: Sequence[QWeight], F: int, mode: int,
               bias: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """act(x Wg^T) * (x Wu^T) -> bf16 [M, F] in ONE tile-GEMM launch with the GLU activation in
    its epilogue (gate and up columns of the same index share a tile), for decode batches.  The
    autotuner times it against the unfused pair (tuned GEMM + activation kernel) once per
    32-row bucket; returns None where the fused kernel does not apply or loses."""
    if not (GLU_FUSE and TILE_GEMM and x.is_cuda and bias is None and mode in GLU_ACTS):
        return None
    M, K = x.shape
    if M > MID_MAX_M or M <= SKINNY_MAX_M:
        # prefill chunks: dequant + hipBLASLt + the activation kernel beats every fused GLU tile
        # at M >= 1024 (gemm_bs.hip's GLU mode included, profiles/r6_gemm_bs.md)
        return None
    pair = _glu_pair(ws, F)
    if pair is None:
        return None
    key = ((M + 31) // 32 * 32, K, F, mode, tuple((w.fmt, w.N) for w in ws))
    if key not in _GLU_CHOICE:
        if not GEMM_AUTOTUNE or torch.cuda.is_current_stream_capturing():
            return None
        out = torch.empty(M, F, dtype=torch.bfloat16, device=x.device)
        t_ref = _time_cold(lambda: act(linear_multi(x, ws), F, mode))
        best, best_t = None, t_ref
        cands = [6, 7, 8] if M > 128 else [7, 12, 14]
        if q32_ok([pair[0]], 9) and pair[0].fmt == pair[2].fmt:
            # (128-row tiles at M > 128 -- 107 / 105, two row tiles to fill the chip -- were timed
            # and never won: r5_glu_bench.log)
            cands += [109, 108, 104] if M > 128 else [109, 108, 107]
        if bs_ok([pair[0], pair[2]]) and pair[0].fmt == pair[2].fmt and F % 4 == 0:
            cands += [200, 203] if M > 128 else [201]
        for t in cands:
            tt = _time_cold(lambda t=t: _run_glu(x, pair, F, mode, t, out))
            if tt < best_t:
                best, best_t = t, tt
        _GLU_CHOICE[key] = best
        if os.environ.get("BENCH_DUMP_GEMM"):
            print(f"glu choice M={M} K={K} F={F} -> {best} ({best_t:.1f} us vs unfused {t_ref:.1f} us)", flush=True)
    tile = _GLU_CHOICE[key]
    if tile is None:
        return None
    out = torch.empty(M, F, dtype=torch.bfloat16, device=x.device)
    _run_glu(x, pair, F, mode, tile, out)
    return out


# ---------------------------------------------------------------------------------------
# Fused elementwise
# ---------------------------------------------------------------------------------------

def add_norm(residual: torch.Tensor, add: Optional[Partial], weight: torch.Tensor,
             bias: Optional[torch.Tensor], eps: float, mode: int = 0,
             out: Optional[torch.Tensor] = None, want_out: bool = True,
             out_f32: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """residual[T,D] (fp32, updated in place) += add;  return norm(residual)*w(+b) as bf16
    (out_f32: also written unrounded, in fp32)."""
    T, D = residual.shape
    if add is not None and (add.M != T or add.N != D):
        raise ValueError(f"add_norm: add {tuple(add.t.shape)} vs residual {T}x{D}")
    if not residual.is_cuda:
        if add is not None:
            residual += add.dense()
        if not want_out:
            return None
        x = residual
        if mode == 0:
            y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight
        else:
            mu = x.mean(-1, keepdim=True)
            var = (x - mu).pow(2).mean(-1, keepdim=True)
            y = (x - mu) * torch.rsqrt(var + eps) * weight
            if bias is not None:
                y = y + bias
        if out_f32 is not None:
            out_f32.copy_(y)
        return y.to(torch.bfloat16)
    assert residual.dtype == torch.float32 and residual.is_contiguous()
    if want_out and out is None:
        out = torch.empty(T, D, dtype=torch.bfloat16, device=residual.device)
    a = add.src_args() if add is not None else (None, 0, 0, None)
    _check(lib().la_add_norm(residual.data_ptr(), a[0], a[1], a[2], a[3], int(add is not None),
                             weight.data_ptr(), _ptr(bias), _ptr(out) if want_out else None, T, D,
                             float(eps), mode, _ptr(out_f32), _stream()), "la_add_norm")
    return out if want_out else None


NORM_ROUTER = os.environ.get("LOCALAI_AMD_NORM_ROUTER", "1") == "1"


def add_norm_router(residual: torch.Tensor, add: Optional["Partial"], weight: torch.Tensor,
                    bias: Optional[torch.Tensor], eps: float, mode: int, router: torch.Tensor, topk: int,
                    renorm: bool, scale: float = 1.0, ep_base: int = 0, ep_local: int = 0):
    """add_norm + moe_router in one launch (elementwise.hip add_norm_router_kernel): returns
    (xn bf16 [T, D], ids [T, topk] int32, wts [T*topk] fp32) -- the router reads the bf16-rounded
    normed row, like moe_router on add_norm's output -- or None when the fused kernel does not
    apply (CPU, E > 64, D > 8192); the caller then runs the two ops."""
    T, D = residual.shape
    E = router.shape[0]
    if (not NORM_ROUTER or not residual.is_cuda or E > 64 or topk > min(16, E) or D % 4 or D > 8192
            or router.dtype != torch.float32 or not router.is_contiguous() or router.shape[1] != D):
        return None
    if add is not None and (add.M != T or add.N != D):
        raise ValueError(f"add_norm_router: add {tuple(add.t.shape)} vs residual {T}x{D}")
    assert residual.dtype == torch.float32 and residual.is_contiguous()
    out = torch.empty(T, D, dtype=torch.bfloat16, device=residual.device)
    ids = torch.empty(T, topk, dtype=torch.int32, device=residual.device)
    wts = torch.empty(T * topk, dtype=torch.float32, device=residual.device)
    a = add.src_args() if add is not None else (None, 0, 0, None)
    _check(lib().la_add_norm_router(residual.data_ptr(), a[0], a[1], a[2], a[3], int(add is not None),
                                    weight.data_ptr(), _ptr(bias), out.data_ptr(), T, D, float(eps), mode,
                                    router.data_ptr(), E, topk, int(renorm), float(scale), ep_base,
                                    ep_local or E, ids.data_ptr(), wts.data_ptr(), _stream()), "la_add_norm_router")
    return out, ids, wts


def rope_cos_sin(max_pos: int, rot_dim: int, theta: float, device, freq_scale: float = 1.0,
                 freq_factors: Optional[torch.Tensor] = None, rope_type: str = "none",
                 yarn: Optional[dict] = None) -> torch.Tensor:
    """[max_pos, rot/2, 2] (cos, sin) table, fp32, computed in float64 on the host."""
    half = rot_dim // 2
    inv = 1.0 / (theta ** (np.arange(0, half, dtype=np.float64) * 2.0 / rot_dim))
    if freq_factors is not None:
        inv = inv / freq_factors.detach().cpu().double().numpy()[:half]
    mscale = 1.0
    if rope_type == "yarn" and yarn:
        # YaRN (ggml rope_yarn): blend interpolated/extrapolated frequencies by ramp
        orig = yarn.get("orig_ctx", 4096)
        bf, bs = yarn.get("beta_fast", 32.0), yarn.get("beta_slow", 1.0)
        ext = yarn.get("ext_factor", 1.0)
        def corr_dim(nrot):
            return rot_dim * math.log(orig / (nrot * 2 * math.pi)) / (2 * math.log(theta))
        lo = max(0.0, math.floor(corr_dim(bf)))
        hi = min(rot_dim - 1.0, math.ceil(corr_dim(bs)))
        i = np.arange(half, dtype=np.float64)
        ramp = np.clip((i - lo) / max(0.001, hi - lo), 0, 1)
        mix = (1 - ramp) * ext
        inv = inv * freq_scale * (1 - mix) + inv * mix
        mscale = yarn.get("attn_factor", 1.0) * (1.0 + 0.1 * math.log(1.0 / freq_scale)) if freq_scale < 1 else \
            yarn.get("attn_factor", 1.0)
    else:
        inv = inv * freq_scale
    pos = np.arange(max_pos, dtype=np.float64)
    ang = np.outer(pos, inv)
    cs = np.stack([np.cos(ang) * mscale, np.sin(ang) * mscale], -1).astype(np.float32)
    return torch.from_numpy(cs).to(device)


def rope_kv(qkv: Partial, pos: torch.Tensor, slots: Optional[torch.Tensor], cos_sin: torch.Tensor,
            Hq: int, Hkv: int, Dh: int, rot: int, mode: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
            block_size: int, q_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate q,k; write k,v into the paged cache at `slots`; return q [T,Hq,Dh] bf16."""
    T = qkv.M
    W = (Hq + 2 * Hkv) * Dh
    if qkv.N != W:
        raise ValueError(f"rope_kv: qkv width {qkv.N} != {W}")
    if not qkv.t.is_cuda:
        x = qkv.dense().view(T, Hq + 2 * Hkv, Dh)
        cs = cos_sin[pos.long()]  # [T, rot/2, 2]
        c, s = cs[..., 0], cs[..., 1]

        def rot_fn(h):
            h = h.clone()
            if mode == 0:
                x0, x1 = h[..., 0:rot:2].clone(), h[..., 1:rot:2].clone()
                h[..., 0:rot:2] = x0 * c[:, None] - x1 * s[:, None]
                h[..., 1:rot:2] = x0 * s[:, None] + x1 * c[:, None]
            else:
                half = rot // 2
                x0, x1 = h[..., :half].clone(), h[..., half:rot].clone()
                h[..., :half] = x0 * c[:, None] - x1 * s[:, None]
                h[..., half:rot] = x0 * s[:, None] + x1 * c[:, None]
            return h
        q = rot_fn(x[:, :Hq]).to(torch.bfloat16)
        k = rot_fn(x[:, Hq:Hq + Hkv]).to(k_cache.dtype)
        v = x[:, Hq + Hkv:].to(v_cache.dtype)
        if slots is not None:
            sl = slots.long()
            ok = sl >= 0
            blk, off = sl[ok] // block_size, sl[ok] % block_size
            k_cache[blk, :, off] = k[ok]
            v_cache[blk, :, off // 8, :, off % 8] = v[ok]
        if q_out is not None:
            q_out.copy_(q)
            return q_out
        return q
    if q_out is None:
        q_out = torch.empty(T, Hq, Dh, dtype=torch.bfloat16, device=qkv.t.device)
    a = qkv.src_args()
    _check(lib().la_rope_kv(a[0], a[1], a[2], a[3], pos.data_ptr(), _ptr(slots), cos_sin.data_ptr(), T, Hq, Hkv,
                            Dh, rot, mode, q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_size,
                            _stream()), "la_rope_kv")
    return q_out


ACT_SWIGLU, ACT_GELU, ACT_GELU_QUICK, ACT_GEGLU = 0, 1, 2, 3
ACT_RELU2 = 4   # max(x, 0)^2
GLU_ACTS = (ACT_SWIGLU, ACT_GEGLU)  # gate|up sources of width 2F


def act(src: Partial, F: int, mode: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    T = src.M
    if not src.t.is_cuda:
        x = src.dense()
        if mode == ACT_SWIGLU:
            y = torch.nn.functional.silu(x[:, :F]) * x[:, F:2 * F]
        elif mode == ACT_GEGLU:
            y = torch.nn.functional.gelu(x[:, :F], approximate="tanh") * x[:, F:2 * F]
        elif mode == ACT_GELU:
            y = torch.nn.functional.gelu(x, approximate="tanh")
        elif mode == ACT_RELU2:
            y = torch.relu(x).square()
        else:
            y = x * torch.sigmoid(1.702 * x)
        return y.to(torch.bfloat16)
    if out is None:
        out = torch.empty(T, F, dtype=torch.bfloat16, device=src.t.device)
    a = src.src_args()
    _check(lib().la_act(a[0], a[1], a[2], a[3], out.data_ptr(), T, F, mode, _stream()), "la_act")
    return out


def act_linear(src: Partial, F: int, mode: int, w: QWeight) -> Partial:
    """down(act(gate|up)).  On the decode GEMV path (M <= GEMV_MAX_M, fp32 slab source) the
    activation is computed inside the down GEMV's activation prologue -- no activation launch
    and no bf16 round trip; otherwise act() then linear()."""
    M = src.M
    width = 2 * F if mode in GLU_ACTS else F
    if (src.t.is_cuda and src.S >= 1 and src.S <= 16 and GEMV_DP4 and M <= GEMV_MAX_M and w.gemv_ok
            and w.K == F and src.N == width):
        S = _gemv_splits([w], w.K, M)
        out = torch.empty(S, M, w.N, dtype=torch.float32, device=src.t.device)
        gemv_dp4(None, [w], S, out, act_src=src, act_mode=mode)
        return Partial(out)
    return linear(act(src, F, mode), w)


def reduce(src: Partial, dtype=torch.float32, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Sum of the split-K slabs (+ bias) as one dense [M, N] matrix (into `out`, a contiguous
    [M, N] tensor of `dtype`, when given)."""
    if out is not None:
        dtype = out.dtype
        assert out.is_contiguous() and tuple(out.shape) == (src.M, src.N)
    if not src.t.is_cuda:
        d = src.dense().to(dtype)
        if out is None:
            return d
        out.copy_(d)
        return out
    T, N = src.M, src.N
    if out is None:
        out = torch.empty(T, N, dtype=dtype, device=src.t.device)
    a = src.src_args()
    f32 = out.data_ptr() if dtype == torch.float32 else None
    b16 = out.data_ptr() if dtype == torch.bfloat16 else None
    _check(lib().la_reduce_slabs(a[0], a[1], a[2], a[3], T, N, f32, b16, _stream()), "la_reduce_slabs")
    return out


def embed(tokens: torch.Tensor, w: QWeight, scale: float = 1.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    T = tokens.shape[0]
    if not tokens.is_cuda:
        return w.dequant_f32()[tokens.long()] * scale
    if out is None:
        out = torch.empty(T, w.K, dtype=torch.float32, device=tokens.device)
    assert tokens.dtype == torch.int32
    _check(lib().la_embed(w.fmt, *w.ptrs(), w.N, w.K, tokens.data_ptr(), T, out.data_ptr(), float(scale),
                          _stream()), "la_embed")
    return out


def gather_rows(src: torch.Tensor, idx: torch.Tensor, fill: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = src[idx[t]] if idx[t] >= 0 else fill: one launch (elementwise.hip gather_rows_kernel).
    src [R, C] contiguous, idx int64 [T] on the same device, fill [C] (needed when idx has -1s)."""
    T, C = idx.shape[0], src.shape[1]
    if not src.is_cuda:
        out = src[idx.clamp(min=0)]
        if fill is not None:
            out[idx < 0] = fill.to(out.dtype)
        return out
    assert src.is_contiguous() and idx.dtype == torch.int64 and idx.device == src.device
    out = torch.empty(T, C, dtype=src.dtype, device=src.device)
    if fill is not None:
        fill = fill.to(src.dtype).contiguous()
    _check(lib().la_gather_rows(src.data_ptr(), idx.data_ptr(), T, _ptr(fill), out.data_ptr(),
                                C * src.element_size(), _stream()), "la_gather_rows")
    return out


# ---------------------------------------------------------------------------------------
# Attention
# ---------------------------------------------------------------------------------------

DEC_TARGET_WAVES = 2048  # ~16 waves per CU over 256 CUs
# (sequence, kv head) pairs for which attn_decode runs single-wave workgroups: 2048 of them
# (decode batch 256 x 8 kv heads) are resident at once at 2 waves per SIMD, so every workgroup's
# latency chain (seq_len -> block table -> first K/V tile) starts in ONE residency round, where
# 4-wave workgroups go through 4 rounds.  Measured on MI355X (scripts/attn_bench.py, KV cycled
# through 8 layers' worth of HBM): B=256 x L=384 72.6 vs 74.9 us, B=256 x L=256 equal, but
# B=128 (two partitions per sequence) 50.6 vs 40.2 us and B=512 (two rounds) 119.7 vs 114.0 us,
# hence the window
DEC_NW1_MIN = int(os.environ.get("LOCALAI_AMD_DEC_NW1_MIN", "2048"))
DEC_NW1_MAX = 2048


def decode_waves(B: int, Hkv: int) -> int:
    """Waves per attn_decode workgroup (1 or 4) for a batch of B sequences."""
    return 1 if DEC_NW1_MIN <= B * Hkv <= max(DEC_NW1_MAX, DEC_NW1_MIN) else 4


# B * Hkv up to this: short sequences are split over the grid's partitions too (32-key
# granularity) instead of running as one partition -- a handful of workgroups cannot hide the
# KV load latency at batch 1 (attn_decode's one_part rule, nw bit 8)
DEC_SPLIT_SHORT = int(os.environ.get("LOCALAI_AMD_DEC_SPLIT_SHORT", "0"))


def _dec_split_short(B: int, Hkv: int) -> bool:
    return B * Hkv <= DEC_SPLIT_SHORT


def decode_partitions(B: int, Hkv: int, max_len: int, block_size: int = 32) -> Tuple[int, int]:
    """Split-KV partitioning for attn_decode: (P, PS).  Enough partitions to put ~16 waves on
    every CU; each workgroup (decode_waves waves) covers PS keys (multiple of 128 -- of 32 for
    the few-sequence split -- at most 2048 pages so the partition's block-table slice fits the
    kernel's LDS stage)."""
    max_len = max(1, max_len)
    nw = decode_waves(B, Hkv)
    gran = max(32, block_size) if _dec_split_short(B, Hkv) else 128
    P = max(1, min(-(-DEC_TARGET_WAVES // (B * Hkv * nw)), -(-max_len // gran), 64))
    P = max(P, -(-max_len // (2048 * block_size)))
    PS = -(-(-(-max_len // P)) // gran) * gran
    P = -(-max_len // PS)
    return P, PS


def _dec_nw(B: int, Hkv: int) -> int:
    return decode_waves(B, Hkv) | (256 if _dec_split_short(B, Hkv) else 0)


def decode_workspace(B: int, Hq: int, Hkv: int, Dh: int, max_len: int, device, block_size: int = 32):
    """Persistent buffers for attn_decode (split-KV partials + self-resetting merge tickets)."""
    P, _ = decode_partitions(B, Hkv, max_len, block_size)
    return (torch.empty(max(1, B * Hq * P * Dh), dtype=torch.float32, device=device),
            torch.empty(max(1, B * Hq * P * 2), dtype=torch.float32, device=device),
            torch.zeros(max(1, B * Hkv), dtype=torch.int32, device=device))


def attn_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                seq_lens: torch.Tensor, scale: float, max_seq_len: int, out: Optional[torch.Tensor] = None,
                workspace: Optional[Tuple[torch.Tensor, ...]] = None, softcap: float = 0.0,
                window: int = 0, dist_bias: Optional[torch.Tensor] = None,
                sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [B,Hq,Dh] bf16; K cache [nblk,Hkv,BS,Dh]; V cache (grouped-transposed pages)
    [nblk,Hkv,BS/8,Dh,8]; block_tables [B,maxb] i32; seq_lens [B] i32.  softcap > 0: scores
    softcap * tanh(s / softcap); window > 0: only the last `window` keys are attended (Gemma-2).
    dist_bias (fp32 [N, Hq]) / sink (fp32 [Hq]): a bias per distance and head (constant from row
    N - 1 on) and a logit without key or value in the softmax denominator, as in attn_mix."""
    B, Hq, Dh = q.shape
    nblk, Hkv, BS, Dh2 = k_cache.shape
    if Dh2 != Dh or Hq % Hkv or tuple(v_cache.shape) != (nblk, Hkv, BS // 8, Dh, 8):
        raise ValueError("attn_decode: head/cache shape mismatch")
    if not q.is_cuda:
        if dist_bias is not None or sink is not None:
            raise ValueError("attn_decode: distance bias and sink have no CPU path here (attn_mix has)")
        return _attn_ref_decode(q, k_cache, v_cache, block_tables, seq_lens, scale, softcap, window)
    for t in (dist_bias, sink):
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or not t.is_cuda or t.shape[-1] != Hq):
            raise ValueError("attn_decode: dist_bias [N, Hq] and sink [Hq] are contiguous fp32")
    P, PS = decode_partitions(B, Hkv, max_seq_len, BS)
    if out is None:
        out = torch.empty(B, Hq, Dh, dtype=torch.bfloat16, device=q.device)
    if (workspace is None or len(workspace) < 3 or workspace[0].numel() < B * Hq * P * Dh
            or workspace[1].numel() < B * Hq * P * 2 or workspace[2].numel() < B * Hkv):
        workspace = decode_workspace(B, Hq, Hkv, Dh, max_seq_len, q.device, BS)
    po, pml, tk = workspace[:3]
    _check(lib().la_attn_decode(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(),
                                block_tables.shape[1], seq_lens.data_ptr(), B, Hq, Hkv, Dh, BS, float(scale), P, PS,
                                out.data_ptr(), po.data_ptr(), pml.data_ptr(), tk.data_ptr(), None, 0, 0, None, None,
                                None, None, float(softcap), int(window), _dec_nw(B, Hkv), _ptr(dist_bias),
                                dist_bias.shape[0] if dist_bias is not None else 0, _ptr(sink), _stream()),
           "la_attn_decode")
    return out


# Off by default: measured on MI355X (Llama-3-8B Q4_K_M, engine bench) the fused launch is not
# faster -- C=1 435.5 vs 440.4 tok/s, C=256 26.43k vs 26.55k -- because the q|k|v slab loads move
# onto the attention kernel's critical path instead of disappearing with the rope_kv launch.
FUSED_DECODE_ROPE = os.environ.get("LOCALAI_AMD_FUSED_ROPE", "0") == "1"


def attn_decode_rope(qkv: Partial, pos: torch.Tensor, slots: torch.Tensor, cos_sin: torch.Tensor, Hq: int,
                     Hkv: int, Dh: int, rot: int, mode: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     block_tables: torch.Tensor, seq_lens: torch.Tensor, scale: float, max_seq_len: int,
                     out: Optional[torch.Tensor] = None,
                     workspace: Optional[Tuple[torch.Tensor, ...]] = None, softcap: float = 0.0,
                     window: int = 0) -> torch.Tensor:
    """Decode step attention with the step's RoPE + paged KV append fused into the attention
    kernel (one launch instead of rope_kv + attn_decode).  Same numerics as the two-kernel path
    (q/k rotated in fp32, rounded to bf16).  Falls back to rope_kv + attn_decode for NEOX /
    partial rotary, Dh not a multiple of 32, or CPU tensors."""
    T = qkv.M
    nblk, _, BS, _ = k_cache.shape
    fusable = (FUSED_DECODE_ROPE and qkv.t.is_cuda and mode == 0 and rot == Dh and Dh % 32 == 0
               and k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16
               and qkv.N == (Hq + 2 * Hkv) * Dh and (qkv.S >= 1 or qkv.t.dtype == torch.bfloat16)
               and tuple(cos_sin.shape[1:]) == (Dh // 2, 2))
    if not fusable:
        q = rope_kv(qkv, pos, slots, cos_sin, Hq, Hkv, Dh, rot, mode, k_cache, v_cache, BS)
        return attn_decode(q, k_cache, v_cache, block_tables, seq_lens, scale, max_seq_len, out=out,
                           workspace=workspace, softcap=softcap, window=window)
    if Hq % Hkv or tuple(v_cache.shape) != (nblk, Hkv, BS // 8, Dh, 8) or k_cache.shape[3] != Dh:
        raise ValueError("attn_decode_rope: head/cache shape mismatch")
    P, PS = decode_partitions(T, Hkv, max_seq_len, BS)
    if out is None:
        out = torch.empty(T, Hq, Dh, dtype=torch.bfloat16, device=qkv.t.device)
    if (workspace is None or len(workspace) < 3 or workspace[0].numel() < T * Hq * P * Dh
            or workspace[1].numel() < T * Hq * P * 2 or workspace[2].numel() < T * Hkv):
        workspace = decode_workspace(T, Hq, Hkv, Dh, max_seq_len, qkv.t.device, BS)
    po, pml, tk = workspace[:3]
    a = qkv.src_args()
    _check(lib().la_attn_decode(None, k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(),
                                block_tables.shape[1], seq_lens.data_ptr(), T, Hq, Hkv, Dh, BS, float(scale), P, PS,
                                out.data_ptr(), po.data_ptr(), pml.data_ptr(), tk.data_ptr(), a[0], a[1], a[2], a[3],
                                pos.data_ptr(), slots.data_ptr(), cos_sin.data_ptr(), float(softcap), int(window),
                                _dec_nw(T, Hkv), None, 0, None, _stream()),
           "la_attn_decode(rope)")
    return out


def v_pages(nblk: int, Hkv: int, BS: int, Dh: int, dtype=torch.bfloat16, device=None) -> torch.Tensor:
    """An empty V cache in the kernels' layout: [nblk, Hkv, BS/8, Dh, 8]."""
    return torch.zeros(nblk, Hkv, BS // 8, Dh, 8, dtype=dtype, device=device)


def v_from_rows(v: torch.Tensor) -> torch.Tensor:
    """[nblk, Hkv, BS, Dh] (key-major pages) -> the V cache layout [nblk, Hkv, BS/8, Dh, 8]."""
    n, h, bs, d = v.shape
    return v.view(n, h, bs // 8, 8, d).transpose(3, 4).contiguous()


def _gather_kv(cache, bt_row, L, transposed=False):
    """-> [Hkv, L, Dh] from K pages [nblk,Hkv,BS,Dh] or V pages [nblk,Hkv,BS/8,Dh,8]."""
    if transposed:
        n, h, g, d, e = cache.shape
        cache = cache.transpose(3, 4).reshape(n, h, g * e, d)
    BS = cache.shape[2]
    nb = (L + BS - 1) // BS
    blocks = cache[bt_row[:nb].long()]                  # [nb, Hkv, BS, Dh]
    return blocks.permute(1, 0, 2, 3).reshape(cache.shape[1], nb * BS, cache.shape[3])[:, :L]


def _softcap_window(s, softcap, window, qpos, kpos):
    """Gemma-2 score transforms of the CPU references: soft-capping, then the sliding window."""
    if softcap > 0:
        s = softcap * torch.tanh(s / softcap)
    if window > 0:
        s = s.masked_fill(qpos - kpos >= window, float("-inf"))
    return s


def _attn_ref_decode(q, kc, vc, bt, sl, scale, softcap=0.0, window=0):
    B, Hq, Dh = q.shape
    Hkv = kc.shape[1]
    G = Hq // Hkv
    out = torch.empty_like(q)
    for b in range(B):
        L = int(sl[b])
        k = _gather_kv(kc, bt[b], L).float()
        v = _gather_kv(vc, bt[b], L, transposed=True).float()
        qq = q[b].float().view(Hkv, G, Dh)
        s = torch.einsum("hgd,hld->hgl", qq, k) * scale
        s = _softcap_window(s, softcap, window, torch.tensor(L - 1), torch.arange(L))
        p = torch.softmax(s, -1)
        out[b] = torch.einsum("hgl,hld->hgd", p, v).reshape(Hq, Dh).to(q.dtype)
    return out


PF_QT = 64


def prefill_tiles(q_lens: Sequence[int], device) -> torch.Tensor:
    tiles = []
    for s, ql in enumerate(q_lens):
        for r in range(0, ql, PF_QT):
            tiles.append((s, r))
    return torch.tensor(tiles, dtype=torch.int32, device=device).view(-1, 2)


def attn_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cu_q: torch.Tensor,
                 ctx_lens: torch.Tensor, block_tables: torch.Tensor, scale: float,
                 tiles: Optional[torch.Tensor] = None, q_lens: Optional[Sequence[int]] = None,
                 out: Optional[torch.Tensor] = None, softcap: float = 0.0, window: int = 0,
                 dist_bias: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention for new tokens. q [T,Hq,Dh]; cu_q [nseq+1]; ctx_lens [nseq] (cached+new).
    dist_bias (fp32 [N, Hq]) / sink (fp32 [Hq]): as in attn_decode and attn_mix."""
    T, Hq, Dh = q.shape
    Hkv = k_cache.shape[1]
    if not q.is_cuda:
        if dist_bias is not None or sink is not None:
            raise ValueError("attn_prefill: distance bias and sink have no CPU path here (attn_mix has)")
        return _attn_ref_prefill(q, k_cache, v_cache, cu_q, ctx_lens, block_tables, scale, softcap, window)
    for t in (dist_bias, sink):
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or not t.is_cuda or t.shape[-1] != Hq):
            raise ValueError("attn_prefill: dist_bias [N, Hq] and sink [Hq] are contiguous fp32")
    if tiles is None:
        cq = cu_q.cpu().tolist()
        tiles = prefill_tiles([cq[i + 1] - cq[i] for i in range(len(cq) - 1)], q.device)
    if out is None:
        out = torch.empty(T, Hq, Dh, dtype=torch.bfloat16, device=q.device)
    _check(lib().la_attn_prefill(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), tiles.data_ptr(),
                                 tiles.shape[0], cu_q.data_ptr(), ctx_lens.data_ptr(), block_tables.data_ptr(),
                                 block_tables.shape[1], Hq, Hkv, Dh, k_cache.shape[2], float(scale),
                                 out.data_ptr(), float(softcap), int(window), _ptr(dist_bias),
                                 dist_bias.shape[0] if dist_bias is not None else 0, _ptr(sink), _stream()), "la_attn_prefill")
    return out


_DENSE_META: Dict[tuple, tuple] = {}


def attn_dense(qkv: torch.Tensor, n: int, L: int, H: int, scale: Optional[float] = None,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Non-causal self-attention of n sequences of L tokens, read in place from a fused q|k|v
    projection output [n * L, 3 * D] (bf16; D = H * Dh): the MFMA flash-attention kernel of
    la_attn_prefill in its dense mode (vision towers).  Returns [n * L, D] bf16."""
    T, W = qkv.shape
    D = W // 3
    Dh = D // H
    if scale is None:
        scale = Dh ** -0.5
    if not qkv.is_cuda:
        q, k, v = qkv.float().view(n, L, 3, H, Dh).permute(2, 0, 3, 1, 4)
        o = torch.softmax(q @ k.transpose(-1, -2) * scale, -1) @ v
        return o.transpose(1, 2).reshape(T, D).to(qkv.dtype)
    if qkv.dtype != torch.bfloat16 or not qkv.is_contiguous() or T != n * L or W != 3 * D:
        raise ValueError("attn_dense: qkv must be a contiguous bf16 [n * L, 3 * D] matrix")
    key = (n, L, qkv.device)
    meta = _DENSE_META.get(key)
    if meta is None:
        cu = torch.arange(0, (n + 1) * L, L, dtype=torch.int32, device=qkv.device)
        meta = _DENSE_META[key] = (cu, prefill_tiles([L] * n, qkv.device))
    cu, tiles = meta
    if out is None:
        out = torch.empty(T, D, dtype=torch.bfloat16, device=qkv.device)
    base = qkv.data_ptr()
    _check(lib().la_attn_dense(base, W, base + 2 * D, W, base + 4 * D, W, out.data_ptr(), D, tiles.data_ptr(),
                               tiles.shape[0], cu.data_ptr(), H, H, Dh, float(scale), _stream()), "la_attn_dense")
    return out


def _attn_ref_prefill(q, kc, vc, cu_q, ctx_lens, bt, scale, softcap=0.0, window=0):
    T, Hq, Dh = q.shape
    Hkv = kc.shape[1]
    G = Hq // Hkv
    out = torch.empty_like(q)
    cq = cu_q.tolist()
    for s in range(len(cq) - 1):
        a, b = cq[s], cq[s + 1]
        ql = b - a
        if ql == 0:
            continue
        L = int(ctx_lens[s])
        k = _gather_kv(kc, bt[s], L).float().repeat_interleave(G, 0)   # [Hq, L, Dh]
        v = _gather_kv(vc, bt[s], L, transposed=True).float().repeat_interleave(G, 0)
        qq = q[a:b].float().transpose(0, 1)                              # [Hq, ql, Dh]
        sc = torch.einsum("hqd,hld->hql", qq, k) * scale
        qpos = torch.arange(L - ql, L).view(-1, 1)
        kpos = torch.arange(L).view(1, -1)
        sc = _softcap_window(sc, softcap, window, qpos, kpos)
        sc = sc.masked_fill(kpos > qpos, float("-inf"))
        p = torch.softmax(sc, -1)
        out[a:b] = torch.einsum("hql,hld->hqd", p, v).transpose(0, 1).to(q.dtype)
    return out


# ---------------------------------------------------------------------------------------
# Short causal convolution on q | k | v + paged K/V append; score-modifier attention
# ---------------------------------------------------------------------------------------

def kv_pages(nblk: int, G: int, BS: int, D: int, dtype=torch.bfloat16, device=None) -> torch.Tensor:
    """Row-major K pages [blocks, G, BS, D] of any dtype (shortconv_kv writes them, attn_mix reads
    them; their V pages are v_pages)."""
    return torch.zeros(nblk, G, BS, D, dtype=dtype, device=device)


def shortconv_kv(u: torch.Tensor, w: torch.Tensor, Cq: int, Ck: int, Cv: int, row_seq: torch.Tensor,
                 cu_q: torch.Tensor, pos: torch.Tensor, slots: torch.Tensor, sslot: torch.Tensor,
                 state: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 vfirst_in: Optional[torch.Tensor] = None, vfirst_out: Optional[torch.Tensor] = None,
                 lam: Optional[torch.Tensor] = None, single: bool = False,
                 w_t: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Depthwise causal convolution over time (w [C, taps] fp32, C = Cq + Ck + Cv; w_t: the same
    weights tap-major, [taps, C], which the vectorised bf16 kernel reads -- made per call when not given) on the first C
    columns of the projection rows u [T, >= C]; rows of one sequence portion are consecutive
    (row_seq [T] -> sequence, cu_q [nseq + 1] row ranges, pos [T] positions).  What precedes a
    portion comes from state[sslot[seq]] ([slots, taps - 1, C]: the last taps - 1 projected rows),
    zeros before position 0; the state then advances to the end of the portion.  Returns q [T, Cq];
    k and v go to the paged pools (K: kv_pages [blocks, G, BS, Dk]; V: v_pages, transposed per 8 keys,
    [blocks, G, BS / 8, Dv, 8]) at `slots` (-1: nowhere), v first mixed
    as (1 - lam) v + lam vfirst_in when given; vfirst_out receives the unmixed v (fp32 [T, Cv]).
    single: every sequence brings one row (decode batches): one fused launch."""
    T = u.shape[0]
    C = Cq + Ck + Cv
    taps = w.shape[1]
    nseq = cu_q.shape[0] - 1
    G, BS, Dk = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    Dv = v_cache.shape[3]
    if v_cache.dim() != 5 or v_cache.shape[2] * 8 != BS or v_cache.shape[4] != 8:
        raise ValueError("shortconv_kv: V pages must be [blocks, G, BS / 8, Dv, 8]")
    if (w.shape[0] != C or u.shape[1] < C or Ck != G * Dk or Cv != G * Dv or state.shape[1:] != (max(taps - 1, 0), C)
            or row_seq.shape[0] != T or pos.shape[0] != T or slots.shape[0] != T or sslot.shape[0] != nseq):
        raise ValueError("shortconv_kv: operand shapes do not fit")
    if single and nseq != T:
        raise ValueError("shortconv_kv: single needs one row per sequence")
    if not u.is_cuda:
        uf = u[:, :C].float()
        y = torch.zeros(T, C)
        cu = cu_q.tolist()
        for s in range(nseq):
            a, b = cu[s], cu[s + 1]
            if b <= a:
                continue
            ss = int(sslot[s])
            p0 = int(pos[a])
            hist = torch.zeros(taps - 1, C)
            if ss >= 0 and taps > 1:
                hist = state[ss].float().clone()
                for i in range(taps - 1):            # state row i holds position p0 - (taps - 1) + i
                    if p0 - (taps - 1) + i < 0:
                        hist[i] = 0
            ext = torch.cat([hist, uf[a:b]], 0)
            for j in range(taps):
                y[a:b] += w[:, j].float() * ext[j:j + (b - a)]
            if ss >= 0 and taps > 1:
                state[ss] = ext[-(taps - 1):].to(state.dtype)
        q = y[:, :Cq].to(u.dtype)
        k = y[:, Cq:Cq + Ck]
        v = y[:, Cq + Ck:]
        if vfirst_out is not None:
            vfirst_out.copy_(v)
        if vfirst_in is not None:
            v = (1.0 - lam.float()) * v + lam.float() * vfirst_in
        sl = slots.long()
        ok = sl >= 0
        blk, off = sl[ok] // BS, sl[ok] % BS
        k_cache[blk, :, off] = k[ok].view(-1, G, Dk).to(k_cache.dtype)
        v_cache[blk, :, off // 8, :, off % 8] = v[ok].view(-1, G, Dv).to(v_cache.dtype)
        return q
    f32 = u.dtype == torch.float32
    if u.dtype not in (torch.float32, torch.bfloat16) or any(t.dtype != u.dtype for t in (state, k_cache, v_cache)):
        raise ValueError("shortconv_kv: projection, state and caches share one dtype (bf16 or fp32)")
    if u.stride(1) != 1 or w.dtype != torch.float32 or not w.is_contiguous() or not state.is_contiguous():
        raise ValueError("shortconv_kv: bad strides")
    for t in (row_seq, cu_q, pos, slots, sslot):
        assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous()
    for t in (vfirst_in, vfirst_out):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == (T, Cv))
    assert (vfirst_in is None) == (lam is None) and (lam is None or lam.dtype == torch.float32)
    q = torch.empty(T, Cq, dtype=u.dtype, device=u.device)
    if w_t is None and not f32:
        w_t = w.t().contiguous()
    if w_t is not None and (w_t.dtype != torch.float32 or tuple(w_t.shape) != (taps, C) or not w_t.is_contiguous()):
        raise ValueError("shortconv_kv: w_t must be the fp32 [taps, C] transpose of w")
    _check(lib().la_shortconv_kv(int(f32), int(single), u.data_ptr(), u.stride(0), w.data_ptr(), _ptr(w_t), taps, Cq, Ck, Cv,
                                 row_seq.data_ptr(), cu_q.data_ptr(), pos.data_ptr(), slots.data_ptr(),
                                 sslot.data_ptr(), state.data_ptr(), q.data_ptr(), k_cache.data_ptr(),
                                 v_cache.data_ptr(), G, Dk, Dv, BS, _ptr(vfirst_in), _ptr(vfirst_out), _ptr(lam), T,
                                 nseq, _stream()), "la_shortconv_kv")
    return q


def alibi_slopes(H: int, device=None) -> torch.Tensor:
    """Per-head distance slopes 2^(-8 (h + 1) / H), fp32 [H]."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=torch.float32, device=device)


ATTN_MIX_QT = 16   # query rows per tile of the matrix-core kernel
ATTN_MIX_TILES = os.environ.get("LOCALAI_AMD_ATTN_MIX_TILES", "1") == "1"


def attn_mix_tiles(q_lens: Sequence[int], device) -> Tuple[torch.Tensor, int]:
    """Work tiles of attn_mix's matrix-core kernel for the leading sequences of a batch, whose
    portions hold q_lens rows: ([ntiles, 2] int32 (sequence, first row within its portion), rows
    covered)."""
    t = [(s, r) for s, n in enumerate(q_lens) for r in range(0, int(n), ATTN_MIX_QT)]
    return torch.tensor(t or [(0, 0)], dtype=torch.int32, device=device), int(sum(int(n) for n in q_lens))


def attn_mix(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, row_seq: torch.Tensor, pos: torch.Tensor,
             block_tables: torch.Tensor, H: int, scale: float, softcap: float = 0.0,
             slopes: Optional[torch.Tensor] = None, talk: Optional[torch.Tensor] = None, chunk: int = 0,
             window: int = 0, gate: Optional[torch.Tensor] = None, tiles: Optional[torch.Tensor] = None,
             tile_rows: int = 0, cu_q: Optional[torch.Tensor] = None, key_splits: int = 1,
             v_width: int = 0, dist_bias: Optional[torch.Tensor] = None,
             sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention with reshaped scores over paged K ([blocks, G, BS, Dk]) and V ([blocks, G, BS / 8,
    Dv, 8], transposed per 8 keys: the operand layout of the P.V matrix instruction); one
    query row per token, row r belonging to sequence row_seq[r] (block_tables row) at position
    pos[r], its keys 0..pos[r] already in the pools.  Per head g: s = scale q.k, softcap tanh,
    minus slopes[g] * distance; then the heads' scores are mixed by talk [H, H]; keys are visible
    within the query's chunk of `chunk` positions and the last `window` positions (0: no limit);
    softmax; values of width Dv; each head's output times sigmoid(gate[r, h]) (gate: [T, H] view,
    any row stride).  Returns [T, H * Dv] in q's dtype; scores and softmax in fp32.
    tiles / tile_rows / cu_q (attn_mix_tiles): the first tile_rows rows are whole prompt portions,
    positions consecutive within each; in bf16 and where the shape allows (key width % 32, value
    width % 16 and <= 128, at most 32 heads) they run on the matrix-core tile kernel, every other
    row -- fp32, odd shapes, rows after tile_rows -- on the row kernel.  key_splits > 1 deals every
    tile's keys to that many workgroups and merges their partial results in a second launch: for
    batches of few rows with many keys each (decoding).
    v_cache None with v_width > 0: a key row's first v_width columns are also its value (latent
    caches, where one stored row serves as key and value); in bf16 with one kv head, key width % 32
    and value width % 32 such calls run on the latent matrix-core kernel (key_splits as above),
    else on the row kernel.
    dist_bias (fp32 [N, H]): dist_bias[min(i - j, N - 1), h] is added to head h's score of key j
    after scale and softcap (a learned bias per distance, constant from N - 1 on; see
    bucketed_bias).  sink (fp32 [H]): the softmax denominator of head h also holds exp(sink[h]),
    a logit without key or value that counts once per query.  Both need talk None."""
    T = q.shape[0]
    G, BS, Dk = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    if (dist_bias is not None or sink is not None) and (talk is not None or v_cache is None):
        raise ValueError("attn_mix: distance bias and sink are not combined with the head mix or latent caches")
    if dist_bias is not None and (dist_bias.dim() != 2 or dist_bias.shape[1] != H or dist_bias.shape[0] < 1):
        raise ValueError("attn_mix: dist_bias is [N, H]")
    if sink is not None and sink.numel() != H:
        raise ValueError("attn_mix: sink is [H]")
    if v_cache is None:
        if not 0 < v_width <= Dk:
            raise ValueError("attn_mix: without V pages v_width names the value columns of a key row")
        Dv = int(v_width)
    else:
        Dv = v_cache.shape[3]
        if v_cache.dim() != 5 or v_cache.shape[2] * 8 != BS or v_cache.shape[4] != 8:
            raise ValueError("attn_mix: V pages must be [blocks, G, BS / 8, Dv, 8]")
    if q.shape[1] != H * Dk or H % G or row_seq.shape[0] != T or pos.shape[0] != T:
        raise ValueError("attn_mix: operand shapes do not fit")
    if not q.is_cuda:
        out = torch.zeros(T, H, Dv)
        rep = H // G
        qf = q.float().view(T, H, Dk)
        for r in range(T):
            i = int(pos[r])
            lo = (i // chunk) * chunk if chunk > 0 else 0
            if window > 0:
                lo = max(lo, i - window + 1)
            js = torch.arange(lo, i + 1)
            tab = block_tables[int(row_seq[r])].long()
            blk, off = tab[js // BS], js % BS
            kk = k_cache[blk, :, off].float().repeat_interleave(rep, 1)     # [n, H, Dk]
            if v_cache is None:
                vv = kk[..., :Dv]
            else:
                vv = v_cache[blk, :, off // 8, :, off % 8].float().repeat_interleave(rep, 1)
            s = torch.einsum("hd,nhd->hn", qf[r], kk) * scale
            if softcap > 0:
                s = softcap * torch.tanh(s / softcap)
            if slopes is not None:
                s = s - slopes.float().view(H, 1) * (i - js).float().view(1, -1)
            if talk is not None:
                s = talk.float() @ s
            if dist_bias is not None:
                s = s + dist_bias.float()[(i - js).clamp(max=dist_bias.shape[0] - 1)].t()
            if sink is not None:    # one more logit in the denominator, nothing in the numerator
                pr = torch.softmax(torch.cat([s, sink.float().view(H, 1)], 1), -1)[:, :-1]
            else:
                pr = torch.softmax(s, -1)
            o = torch.einsum("hn,nhd->hd", pr, vv)
            if gate is not None:
                o = o * torch.sigmoid(gate[r].float()).view(H, 1)
            out[r] = o
        return out.view(T, H * Dv).to(q.dtype)
    f32 = q.dtype == torch.float32
    if (q.dtype not in (torch.float32, torch.bfloat16) or k_cache.dtype != q.dtype
            or (v_cache is not None and v_cache.dtype != q.dtype)):
        raise ValueError("attn_mix: q and the caches share one dtype (bf16 or fp32)")
    if not (q.is_contiguous() and k_cache.is_contiguous() and (v_cache is None or v_cache.is_contiguous())
            and block_tables.is_contiguous()):
        raise ValueError("attn_mix: operands must be contiguous")
    for t in (row_seq, pos, block_tables):
        assert t.dtype == torch.int32 and t.is_cuda
    for t in (slopes, talk, dist_bias, sink):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda)
    assert slopes is None or slopes.numel() == H
    nbias = dist_bias.shape[0] if dist_bias is not None else 0
    assert talk is None or tuple(talk.shape) == (H, H)
    ldg = 0
    if gate is not None:
        if gate.dtype != q.dtype or tuple(gate.shape) != (T, H) or gate.stride(1) != 1:
            raise ValueError("attn_mix: gate must be a [T, H] view of q's dtype with unit column stride")
        ldg = gate.stride(0)
    out = torch.empty(T, H * Dv, dtype=q.dtype, device=q.device)
    r0 = 0
    if (v_cache is None and not f32 and G == 1 and ATTN_MIX_TILES and softcap == 0.0 and slopes is None and talk is None
            and chunk == 0 and _has("la_attn_latent")):
        # latent caches in bf16: the heads of a token are the rows of a matrix-core tile, the cached
        # rows of a key tile staged once for Q.K^T and P.V (attention_latent.hip)
        ns = max(1, min(int(key_splits), 64))
        po = pml = None
        if ns > 1:
            po = torch.empty(T * H * ns * Dv, dtype=torch.float32, device=q.device)
            pml = torch.empty(T * H * ns * 2, dtype=torch.float32, device=q.device)
        rc = lib().la_attn_latent(q.data_ptr(), k_cache.data_ptr(), row_seq.data_ptr(), pos.data_ptr(),
                                  block_tables.data_ptr(), block_tables.shape[1], T, H, Dk, Dv, BS, float(scale), int(window),
                                  _ptr(gate), ldg, out.data_ptr(), ns, _ptr(po), _ptr(pml), _stream())
        if rc == 0:
            return out
        if rc != 1:
            _check(rc, "la_attn_latent")
    if (tiles is not None and tile_rows > 0 and not f32 and ATTN_MIX_TILES and Dk % 32 == 0 and Dv % 16 == 0
            and Dv <= 128 and H <= 32 and v_cache is not None):
        if cu_q is None or tile_rows > T or tiles.dtype != torch.int32 or not tiles.is_contiguous():
            raise ValueError("attn_mix: tiles need cu_q and int32 [ntiles, 2]")
        ns = max(1, min(int(key_splits), 64))
        po = pml = None
        if ns > 1:
            po = torch.empty(tile_rows * H * ns * Dv, dtype=torch.float32, device=q.device)
            pml = torch.empty(tile_rows * H * ns * 2, dtype=torch.float32, device=q.device)
        rc = lib().la_attn_mix_tiles(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), tiles.data_ptr(),
                                     tiles.shape[0], cu_q.data_ptr(), pos.data_ptr(), block_tables.data_ptr(),
                                     block_tables.shape[1], H, G, Dk, Dv, BS, float(scale), float(softcap), _ptr(slopes),
                                     _ptr(talk), int(chunk), int(window), _ptr(gate), ldg, out.data_ptr(), ns,
                                     _ptr(po), _ptr(pml), tile_rows, _ptr(dist_bias), nbias, _ptr(sink), _stream())
        if rc == 0:
            r0 = tile_rows
        elif rc != 1:
            _check(rc, "la_attn_mix_tiles")
    if r0 < T:
        esz = q.element_size()
        _check(lib().la_attn_mix_rows(int(f32), q.data_ptr() + r0 * H * Dk * esz, k_cache.data_ptr(),
                                      _ptr(v_cache), row_seq.data_ptr() + r0 * 4, pos.data_ptr() + r0 * 4,
                                      block_tables.data_ptr(), block_tables.shape[1], T - r0, H, G, Dk, Dv, BS,
                                      float(scale), float(softcap), _ptr(slopes), _ptr(talk), int(chunk), int(window),
                                      None if gate is None else gate.data_ptr() + r0 * ldg * esz, ldg,
                                      out.data_ptr() + r0 * H * Dv * esz, _ptr(dist_bias), nbias, _ptr(sink), _stream()),
               "la_attn_mix_rows")
    return out


def router_sigmoid(xn: torch.Tensor, router: torch.Tensor, corr: Optional[torch.Tensor], topk: int,
                   renorm: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """Sigmoid-score router: s = sigmoid(xn @ router^T) in fp32; the topk experts with the largest
    s + corr (corr: selection only) are chosen, their weights are s / (sum of the chosen s + 1e-20)
    (renorm) or s.  Returns (ids [T, topk] int32, weights [T * topk] fp32)."""
    T, D = xn.shape
    E = router.shape[0]
    if not xn.is_cuda:
        s = torch.sigmoid(xn.float() @ router.float().t())
        c = s if corr is None else s + corr.float()
        idx = torch.topk(c, topk, -1).indices
        w = s.gather(1, idx)
        if renorm:
            w = w / (w.sum(-1, keepdim=True) + 1e-20)
        return idx.to(torch.int32), w.reshape(-1).float()
    assert xn.dtype in (torch.bfloat16, torch.float32) and xn.stride(1) == 1
    assert router.dtype == torch.float32 and router.is_contiguous() and router.shape[1] == D
    assert corr is None or (corr.dtype == torch.float32 and corr.numel() == E)
    ids = torch.empty(T, topk, dtype=torch.int32, device=xn.device)
    wts = torch.empty(T * topk, dtype=torch.float32, device=xn.device)
    _check(lib().la_router_sigmoid(int(xn.dtype == torch.float32), xn.data_ptr(), xn.stride(0), router.data_ptr(),
                                   _ptr(corr), E, D, T, topk, int(renorm), ids.data_ptr(), wts.data_ptr(), _stream()),
           "la_router_sigmoid")
    return ids, wts


def router_softmax(xn: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor], topk: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Logit router: z = xn @ router^T + bias in fp32; the topk experts with the largest z are
    chosen (ties: lowest expert id) and weighted by the softmax over the chosen logits only.
    Returns (ids [T, topk] int32, weights [T * topk] fp32)."""
    T, D = xn.shape
    E = router.shape[0]
    if not xn.is_cuda:
        z = xn.float() @ router.float().t()
        if bias is not None:
            z = z + bias.float()
        val, idx = torch.topk(z, topk, -1)
        return idx.to(torch.int32), torch.softmax(val, -1).reshape(-1).float()
    assert xn.dtype in (torch.bfloat16, torch.float32) and xn.stride(1) == 1
    assert router.dtype == torch.float32 and router.is_contiguous() and router.shape[1] == D
    assert bias is None or (bias.dtype == torch.float32 and bias.numel() == E and bias.is_contiguous())
    ids = torch.empty(T, topk, dtype=torch.int32, device=xn.device)
    wts = torch.empty(T * topk, dtype=torch.float32, device=xn.device)
    _check(lib().la_router_topk(int(xn.dtype == torch.float32), 1, xn.data_ptr(), xn.stride(0), router.data_ptr(),
                                _ptr(bias), E, D, T, topk, 1, ids.data_ptr(), wts.data_ptr(), _stream()),
           "la_router_topk")
    return ids, wts


def moe_pairs(x: torch.Tensor, wg: torch.Tensor, wu: torch.Tensor, wd: torch.Tensor, ids: torch.Tensor,
              wts: torch.Tensor, clamp: Optional[Tuple[float, float]] = None) -> torch.Tensor:
    """Routed gated experts as (token, expert) pair GEMVs on dense stacked weights (small batches,
    any width, no host sync): y[t] = sum_k wts[t, k] * Wd[e] (silu(Wg[e] x[t]) * (Wu[e] x[t])),
    e = ids[t, k].  wg / wu [E, F, D], wd [E, D, F] in x's dtype (bf16 or fp32).  Returns fp32 [T, D].
    clamp = (limit, slope): the clamped unit of glu_clamp instead of SiLU gating, g = min(Wg x,
    limit), u = clamp(Wu x, -limit, limit), g sigmoid(slope g) (u + 1)."""
    T, D = x.shape
    E, F = wg.shape[0], wg.shape[1]
    topk = ids.shape[1]
    if not x.is_cuda:
        xf = x.float()
        y = torch.zeros(T, D)
        wv = wts.view(T, topk)
        for t in range(T):
            for k in range(topk):
                e = int(ids[t, k])
                g_, u_ = wg[e].float() @ xf[t], wu[e].float() @ xf[t]
                if clamp is None:
                    h = torch.nn.functional.silu(g_) * u_
                else:
                    g_ = torch.clamp(g_, max=clamp[0])
                    h = g_ * torch.sigmoid(clamp[1] * g_) * (torch.clamp(u_, -clamp[0], clamp[0]) + 1.0)
                y[t] += wv[t, k] * (wd[e].float() @ h.to(x.dtype).float())
        return y
    for w_ in (wg, wu, wd):
        assert w_.dtype == x.dtype and w_.is_contiguous()
    assert tuple(wu.shape) == (E, F, D) and tuple(wd.shape) == (E, D, F) and x.is_contiguous()
    assert ids.dtype == torch.int32 and ids.is_contiguous() and wts.dtype == torch.float32
    h = torch.empty(T * topk, F, dtype=x.dtype, device=x.device)
    y = torch.empty(T, D, dtype=torch.float32, device=x.device)
    _check(lib().la_moe_pairs(int(x.dtype == torch.float32), x.data_ptr(), wg.data_ptr(), wu.data_ptr(), wd.data_ptr(),
                              ids.data_ptr(), wts.data_ptr(), T, topk, D, F, E, h.data_ptr(), y.data_ptr(),
                              int(clamp is not None), float(clamp[0]) if clamp else 0.0, float(clamp[1]) if clamp else 0.0,
                              _stream()),
           "la_moe_pairs")
    return y


# ---------------------------------------------------------------------------------------
# Layer-list designs: squashing norms, rotations into pages, latent caches, retention
# ---------------------------------------------------------------------------------------

def _branch_args(b, T: int, N: int):
    """(pointer, is fp32, slab stride, slabs) of a [T, N] GEMM result: a Partial (fp32 split-K
    slabs or one bf16 / fp32 matrix) or a dense contiguous tensor."""
    t = b.t if isinstance(b, Partial) else b
    if isinstance(b, Partial) and b.bias is not None:
        raise ValueError("a biased partial is not taken here")
    if t.shape[-2] != T or t.shape[-1] != N or not t.is_contiguous():
        raise ValueError(f"operand {tuple(t.shape)} does not fit [{T}, {N}]")
    if t.dim() == 3:
        if t.dtype != torch.float32:
            raise ValueError("slab sources are fp32")
        return t.data_ptr(), 1, T * N, t.shape[0]
    if t.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("sources are bf16 or fp32")
    return t.data_ptr(), int(t.dtype == torch.float32), 0, 1


def _branch_dense(b) -> torch.Tensor:
    return b.dense() if isinstance(b, Partial) else b.float()


NORM_NONE, NORM_DYT, NORM_RMS, NORM_CAST, NORM_LN = 0, 1, 2, 3, 4


def _ln_ref(y: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    mu = y.mean(-1, keepdim=True)
    d = y - mu
    return d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w.float()


def norm_chain(res: torch.Tensor, branch=None, post: Optional[tuple] = None, pre: Optional[tuple] = None,
               add_vec: Optional[torch.Tensor] = None, replace: bool = False,
               out_dtype: torch.dtype = torch.bfloat16) -> Optional[torch.Tensor]:
    """One launch per sublayer boundary of a post-normed residual stream (fp32 [T, D], updated in
    place):  res <- (0 if replace else res) + post(branch) + add_vec, then returns pre(res).
    post / pre:  ("dyt", alpha, w, b): tanh(alpha x) * w + b, a norm without statistics (alpha a
    Python float, w / b fp32 [D]);  ("rms", w, eps): x / sqrt(mean(x^2) + eps) * w (post only);
    ("ln", w, eps): (x - mean) / sqrt(mean((x - mean)^2) + eps) * w, a layer norm without bias (post
    and pre);  ("cast",): res in out_dtype (pre only);  None: identity for post, no output for pre.
    branch: a Partial or dense [T, D] tensor (None: the stream is only read).  All arithmetic fp32."""
    T, D = res.shape
    pm = NORM_NONE if post is None else {"dyt": NORM_DYT, "rms": NORM_RMS, "ln": NORM_LN}[post[0]]
    qm = NORM_NONE if pre is None else {"dyt": NORM_DYT, "cast": NORM_CAST, "ln": NORM_LN}[pre[0]]
    if not res.is_cuda:
        if branch is not None:
            y = _branch_dense(branch)
            if pm == NORM_DYT:
                y = torch.tanh(float(post[1]) * y) * post[2].float() + post[3].float()
            elif pm == NORM_RMS:
                y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + float(post[2])) * post[1].float()
            elif pm == NORM_LN:
                y = _ln_ref(y, post[1], float(post[2]))
            if add_vec is not None:
                y = y + add_vec.float()
            if replace:
                res.copy_(y)
            else:
                res += y
        if qm == NORM_DYT:
            return (torch.tanh(float(pre[1]) * res) * pre[2].float() + pre[3].float()).to(out_dtype)
        if qm == NORM_LN:
            return _ln_ref(res, pre[1], float(pre[2])).to(out_dtype)
        return res.to(out_dtype) if qm == NORM_CAST else None
    if res.dtype != torch.float32 or not res.is_contiguous() or out_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("norm_chain: the stream is contiguous fp32; outputs are bf16 or fp32")
    a = _branch_args(branch, T, D) if branch is not None else (None, 0, 0, 0)
    pa, pw, pb, eps = 0.0, None, None, 0.0
    if pm == NORM_DYT:
        pa, pw, pb = float(post[1]), post[2], post[3]
    elif pm in (NORM_RMS, NORM_LN):
        pw, eps = post[1], float(post[2])
    qa, qw_, qb = (float(pre[1]), pre[2], pre[3]) if qm == NORM_DYT else (0.0, None, None)
    if qm == NORM_LN:       # the output norm's eps travels in the slot of the squashing norm's alpha
        qa, qw_ = float(pre[2]), pre[1]
    for t in (pw, pb, qw_, qb, add_vec):
        if t is not None and (t.dtype != torch.float32 or t.numel() != D or not t.is_contiguous()):
            raise ValueError("norm_chain: weights are contiguous fp32 [D]")
    out = torch.empty(T, D, dtype=out_dtype, device=res.device) if qm != NORM_NONE else None
    _check(lib().la_norm_chain(res.data_ptr(), T, D, a[0], a[1], a[2], a[3], pm, pa, _ptr(pw), _ptr(pb), eps,
                               _ptr(add_vec), int(replace), qm, qa, _ptr(qw_), _ptr(qb), _ptr(out),
                               int(out_dtype == torch.float32), _stream()), "la_norm_chain")
    return out


def glu_clamp(src, F: int, limit: float, slope: float = 1.702, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Clamped gated unit on a gate|up projection [T, 2F]:  g = min(gate, limit), u = clamp(up,
    -limit, limit), y = g * sigmoid(slope * g) * (u + 1).  fp32 arithmetic, [T, F] in out_dtype."""
    t = src.t if isinstance(src, Partial) else src
    T = t.shape[-2]
    if t.shape[-1] != 2 * F:
        raise ValueError("glu_clamp: the source is [T, 2F]")
    if not t.is_cuda:
        x = _branch_dense(src)
        g = torch.clamp(x[:, :F], max=limit)
        u = torch.clamp(x[:, F:], -limit, limit)
        return (g * torch.sigmoid(slope * g) * (u + 1.0)).to(out_dtype)
    a = _branch_args(src, T, 2 * F)
    out = torch.empty(T, F, dtype=out_dtype, device=t.device)
    _check(lib().la_glu_clamp(a[0], a[1], a[2], a[3], T, F, float(limit), float(slope), out.data_ptr(),
                              int(out_dtype == torch.float32), _stream()), "la_glu_clamp")
    return out


def side_gate(z, tokens: torch.Tensor, table: torch.Tensor, col0: int, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """gelu_tanh(z[t]) * table[tokens[t], col0 : col0 + n] for a projection z [T, n]: a per-token
    side embedding (bf16 [V, W] table, any column window) gated by a function of the stream."""
    t = z.t if isinstance(z, Partial) else z
    T, n = t.shape[-2], t.shape[-1]
    if col0 < 0 or col0 + n > table.shape[1] or tokens.shape[0] != T:
        raise ValueError("side_gate: the column window does not fit the table")
    if not t.is_cuda:
        e = table[tokens.long(), col0:col0 + n].float()
        return (torch.nn.functional.gelu(_branch_dense(z), approximate="tanh") * e).to(out_dtype)
    if table.dtype != torch.bfloat16 or not table.is_contiguous() or tokens.dtype != torch.int32:
        raise ValueError("side_gate: bf16 table, int32 tokens")
    a = _branch_args(z, T, n)
    out = torch.empty(T, n, dtype=out_dtype, device=t.device)
    _check(lib().la_side_gate(a[0], a[1], a[2], a[3], T, n, tokens.data_ptr(), table.data_ptr(), table.shape[1],
                              int(col0), out.data_ptr(), int(out_dtype == torch.float32), _stream()), "la_side_gate")
    return out


def rot_freqs(dims: int, base: float, scaling: Optional[dict] = None, device=None) -> Tuple[torch.Tensor, float]:
    """(angular frequencies fp32 [dims / 2], magnitude) of a rotation over `dims` dimensions:
    f_i = base^(-2i / dims).  scaling {"factor", "original", "fast", "slow"} (YaRN): with
    d(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor d(fast), 0), hi = min(ceil
    d(slow), dims - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) the frequency is
    f_i / factor * ramp_i + f_i (1 - ramp_i), and cos / sin are scaled by 0.1 ln(factor) + 1.
    Computed in float64 on the host; the kernels form angles position * f_i in fp32."""
    half = dims // 2
    f = np.power(float(base), -2.0 * np.arange(half, dtype=np.float64) / dims)
    mag = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        d_of = lambda turns: dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))  # noqa: E731
        lo = max(math.floor(d_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(d_of(float(scaling["slow"]))), dims - 1)
        ramp = np.clip((np.arange(half, dtype=np.float64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return torch.from_numpy(f.astype(np.float32)).to(device), float(mag)


def _rotate_ref(x: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor, mag: float, rot: int, off: int,
                interleaved: bool) -> torch.Tensor:
    """x [T, n, d] fp32 with dims [off, off + rot) of every head rotated by angle pos * freqs."""
    ang = pos.float()[:, None] * freqs.float()[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    out = x.clone()
    half = rot // 2
    if interleaved:
        u, v = x[..., off:off + rot:2], x[..., off + 1:off + rot:2]
        out[..., off:off + rot:2] = u * c - v * s
        out[..., off + 1:off + rot:2] = v * c + u * s
    else:
        u, v = x[..., off:off + half], x[..., off + half:off + rot]
        out[..., off:off + half] = u * c - v * s
        out[..., off + half:off + rot] = v * c + u * s
    return out


def _page_write_ref(k_cache, v_cache, slots, k, v):
    BS = k_cache.shape[2]
    sl = slots.long()
    ok = sl >= 0
    blk, off = sl[ok] // BS, sl[ok] % BS
    if k is not None:
        k_cache[blk, :, off] = k[ok].to(k_cache.dtype)
    if v is not None:
        v_cache[blk, :, off // 8, :, off % 8] = v[ok].to(v_cache.dtype)


def rope_pages(src: torch.Tensor, H: int, Dq: int, G: int, Dk: int, Dv: int, pos: torch.Tensor,
               slots: Optional[torch.Tensor], freqs: torch.Tensor, mag: float, rot: int, q_off: int = 0,
               interleaved: bool = True, k_cache: Optional[torch.Tensor] = None,
               v_cache: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotary positions on projection rows src [T, H Dq + G Dk + G Dv] (q | k | v, bf16 or fp32):
    dims [q_off, q_off + rot) of every query head and [0, rot) of every key head are rotated by
    the angle pos * freqs[i] (fp32), pairs (2i, 2i + 1) when interleaved, else (i, i + rot / 2),
    cos and sin times mag; the other dims pass.  Returns q [T, H Dq]; rotated keys and the values
    go to the paged pools (K [blocks, G, BS, Dk], V [blocks, G, BS / 8, Dv, 8]) at `slots` (-1:
    nowhere).  G = 0: queries only."""
    T = src.shape[0]
    Cq, Ck, Cv = H * Dq, G * Dk, G * Dv
    if (src.dim() != 2 or src.shape[1] != Cq + Ck + Cv or rot % 2 or q_off + rot > Dq or (G and rot > Dk)
            or freqs.numel() != rot // 2 or pos.shape[0] != T):
        raise ValueError("rope_pages: operand shapes do not fit")
    if G and (k_cache is None or v_cache is None or slots is None or tuple(k_cache.shape[1:]) != (G, k_cache.shape[2], Dk)
              or tuple(v_cache.shape[1:]) != (G, k_cache.shape[2] // 8, Dv, 8)):
        raise ValueError("rope_pages: pools do not fit the key / value widths")
    if not src.is_cuda:
        x = src.float()
        q = _rotate_ref(x[:, :Cq].reshape(T, H, Dq), pos, freqs, mag, rot, q_off, interleaved)
        if G:
            k = _rotate_ref(x[:, Cq:Cq + Ck].reshape(T, G, Dk), pos, freqs, mag, rot, 0, interleaved)
            _page_write_ref(k_cache, v_cache, slots, k, x[:, Cq + Ck:].reshape(T, G, Dv))
        return q.reshape(T, Cq).to(src.dtype)
    f32 = src.dtype == torch.float32
    if src.dtype not in (torch.float32, torch.bfloat16) or not src.is_contiguous():
        raise ValueError("rope_pages: contiguous bf16 or fp32 rows")
    if G and (k_cache.dtype != src.dtype or v_cache.dtype != src.dtype):
        raise ValueError("rope_pages: pools share the rows' dtype")
    assert pos.dtype == torch.int32 and freqs.dtype == torch.float32 and freqs.is_contiguous()
    assert slots is None or (slots.dtype == torch.int32 and slots.shape[0] == T)
    q = torch.empty(T, Cq, dtype=src.dtype, device=src.device)
    _check(lib().la_rope_pages(int(f32), src.data_ptr(), T, H, Dq, G, Dk, Dv, pos.data_ptr(), _ptr(slots),
                               freqs.data_ptr(), float(mag), rot, q_off, int(interleaved), q.data_ptr(),
                               _ptr(k_cache), _ptr(v_cache), k_cache.shape[2] if G else 0, _stream()), "la_rope_pages")
    return q


def latent_kv(src: torch.Tensor, rank: int, norm_w: torch.Tensor, eps: float, pos: torch.Tensor, slots: torch.Tensor,
              freqs: torch.Tensor, mag: float, k_cache: torch.Tensor, interleaved: bool = True) -> None:
    """Latent key/value rows into a one-head pool [blocks, 1, BS, rank + rot]: of a down-projection
    row src[t] = [c (rank) | r (rot)] the latent part is RMS-normed (c / sqrt(mean c^2 + eps) *
    norm_w, fp32) and the rest rotated by pos[t] * freqs; the stored row [norm c | rot r] is key
    and value at once (attn_mix, v_width = rank)."""
    T, W = src.shape
    rot = W - rank
    if (rank <= 0 or rot < 0 or rot % 2 or freqs.numel() != rot // 2 or norm_w.numel() != rank
            or k_cache.shape[1] != 1 or k_cache.shape[3] != W or pos.shape[0] != T or slots.shape[0] != T):
        raise ValueError("latent_kv: operand shapes do not fit")
    if not src.is_cuda:
        x = src.float()
        c = x[:, :rank]
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
        r = _rotate_ref(x[:, rank:].reshape(T, 1, rot), pos, freqs, mag, rot, 0, interleaved).reshape(T, rot)
        _page_write_ref(k_cache, None, slots, torch.cat([c, r], -1).reshape(T, 1, W), None)
        return
    if src.dtype not in (torch.float32, torch.bfloat16) or not src.is_contiguous() or k_cache.dtype != src.dtype:
        raise ValueError("latent_kv: contiguous bf16 or fp32 rows, pool of the same dtype")
    assert pos.dtype == torch.int32 and slots.dtype == torch.int32 and freqs.dtype == torch.float32
    assert norm_w.dtype == torch.float32 and norm_w.is_contiguous()
    _check(lib().la_latent_kv(int(src.dtype == torch.float32), src.data_ptr(), T, rank, rot, norm_w.data_ptr(),
                              float(eps), pos.data_ptr(), slots.data_ptr(), freqs.data_ptr(), float(mag),
                              int(interleaved), k_cache.data_ptr(), k_cache.shape[2], _stream()), "la_latent_kv")


RETENTION_SEG = 128   # rows per segment of a segmented scan (retention.hip RT_SEG)


def retention_state(slots: int, H: int, Dk: int, Dv: int, device=None) -> torch.Tensor:
    """State pool of ops.retention: fp32 [slots, H, Dv, Dk], every head's Dk x Dv state stored
    value-column major (a column's Dk entries contiguous: the kernel's threads own columns)."""
    return torch.zeros(slots, H, Dv, Dk, dtype=torch.float32, device=device)


def retention(src: torch.Tensor, H: int, Dk: int, Dv: int, pos: torch.Tensor, cu_q: torch.Tensor,
              sslots: torch.Tensor, state: torch.Tensor, decay: torch.Tensor, freqs: torch.Tensor, rot: int,
              eps: float, mag: float = 1.0, max_rows: int = 0) -> torch.Tensor:
    """Decayed linear attention over projection rows src [T, 2 H Dk + 2 H Dv] (q | k | v | gate):
    q and k rotated on their first `rot` dims (pairs (i, i + rot / 2), angle pos * freqs[i]), k
    times Dk^-1/2; per head S <- decay_h S + k v^T, o = S^T q (no softmax, no denominator); o
    divided by its root mean square over the head (eps), times silu(gate).  Rows of a sequence
    portion are consecutive (cu_q [nseq + 1]); its state lives in state[sslots[seq]] (fp32,
    retention_state), is taken as zero when the portion starts at position 0 and advanced to the
    portion's end.  Rotation, state, outputs and the norm are fp32.  max_rows: the longest portion
    of the batch when the caller knows it (0: unknown, taken as T); long portions are scanned in
    segments.  Returns [T, H Dv] in src's dtype."""
    T = src.shape[0]
    nseq = cu_q.shape[0] - 1
    Cq, Cv = H * Dk, H * Dv
    if (src.dim() != 2 or src.shape[1] != 2 * Cq + 2 * Cv or tuple(state.shape[1:]) != (H, Dv, Dk) or decay.numel() != H
            or rot % 2 or rot > Dk or freqs.numel() != rot // 2 or sslots.shape[0] != nseq or pos.shape[0] != T):
        raise ValueError("retention: operand shapes do not fit")
    if not src.is_cuda:
        x = src.float()
        q = _rotate_ref(x[:, :Cq].reshape(T, H, Dk), pos, freqs, mag, rot, 0, False)
        k = _rotate_ref(x[:, Cq:2 * Cq].reshape(T, H, Dk), pos, freqs, mag, rot, 0, False) * Dk ** -0.5
        v = x[:, 2 * Cq:2 * Cq + Cv].reshape(T, H, Dv)
        g = x[:, 2 * Cq + Cv:].reshape(T, H, Dv)
        o = torch.zeros(T, H, Dv)
        cu = cu_q.tolist()
        d = decay.float().view(H, 1, 1)
        for s in range(nseq):
            a, b = cu[s], cu[s + 1]
            if b <= a:
                continue
            ss = int(sslots[s])
            S = torch.zeros(H, Dk, Dv) if int(pos[a]) == 0 else state[ss].float().transpose(1, 2).clone()
            for t in range(a, b):
                S = d * S + k[t].unsqueeze(2) * v[t].unsqueeze(1)
                o[t] = torch.einsum("hkv,hk->hv", S, q[t])
            state[ss] = S.transpose(1, 2)
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
        return (o * torch.nn.functional.silu(g)).reshape(T, Cv).to(src.dtype)
    if src.dtype not in (torch.float32, torch.bfloat16) or not src.is_contiguous():
        raise ValueError("retention: contiguous bf16 or fp32 rows")
    if state.dtype != torch.float32 or not state.is_contiguous():
        raise ValueError("retention: the state pool is contiguous fp32")
    for t in (pos, cu_q, sslots):
        assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous()
    assert decay.dtype == torch.float32 and freqs.dtype == torch.float32
    qk = torch.empty(T, 2 * Cq, dtype=torch.float32, device=src.device)      # rotated q | scaled rotated k
    o = torch.empty(T, Cv, dtype=torch.float32, device=src.device)
    out = torch.empty(T, Cv, dtype=src.dtype, device=src.device)
    # long batches scan their portions in segments of RETENTION_SEG rows: room for every segment's state
    max_rows = int(max_rows) if max_rows > 0 else T
    seg = torch.empty((T // RETENTION_SEG + nseq) * H * Dv * Dk, dtype=torch.float32, device=src.device) \
        if (T >= 8 * RETENTION_SEG and max_rows >= 4 * RETENTION_SEG) else None
    _check(lib().la_retention(int(src.dtype == torch.float32), src.data_ptr(), T, nseq, H, Dk, Dv, pos.data_ptr(),
                              cu_q.data_ptr(), sslots.data_ptr(), state.data_ptr(), state.shape[0], decay.data_ptr(),
                              freqs.data_ptr(), float(mag), rot, float(eps), qk.data_ptr(), o.data_ptr(), out.data_ptr(),
                              _ptr(seg), max_rows, _stream()),
           "la_retention")
    return out


# ---------------------------------------------------------------------------------------
# Layer-list designs: additive positions, unit-normed queries and keys, bucketed distance
# bias, state-space scan
# ---------------------------------------------------------------------------------------

def sinusoid_freqs(width: int, base: float = 10000.0, device=None) -> torch.Tensor:
    """Angular frequencies base^(-2i / width), i = 0 .. ceil(width / 2) - 1 (float64 on the host, fp32 out)."""
    n = (width + 1) // 2
    return torch.from_numpy(np.power(float(base), -2.0 * np.arange(n, dtype=np.float64) / width).astype(np.float32)).to(device)


def sinusoid_add(res: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """Additive sinusoidal positions on an fp32 stream [T, D], in place: column 2i gets
    sin(pos * freqs[i]), column 2i + 1 cos of the same angle (angles formed and evaluated in fp32)."""
    T, D = res.shape
    if freqs.numel() != (D + 1) // 2 or pos.shape[0] != T or res.dtype != torch.float32:
        raise ValueError("sinusoid_add: operand shapes do not fit")
    if not res.is_cuda:
        ang = pos.float()[:, None] * freqs.float()[None, :]
        pe = torch.stack([torch.sin(ang), torch.cos(ang)], -1).reshape(T, -1)[:, :D]
        res += pe
        return res
    assert res.is_contiguous() and pos.dtype == torch.int32 and freqs.dtype == torch.float32 and freqs.is_contiguous()
    _check(lib().la_sinusoid_add(res.data_ptr(), T, D, pos.data_ptr(), freqs.data_ptr(), _stream()), "la_sinusoid_add")
    return res


def bucketed_bias(rel: torch.Tensor, max_dist: int) -> torch.Tensor:
    """Distance-bias table for attn_mix from a learned bucket table rel [B, H]: row n, n = 0 ..
    max_dist, is rel[bucket(n)] with h = B // 2 exact buckets for n < h and B - h logarithmic ones
    up to max_dist: bucket(n) = min(B - 1, h + floor(ln(n / h) / ln(max_dist / h) * (B - h))).  From
    max_dist on the bucket is B - 1, so attn_mix's clamp at the last row is exact.  fp32 [max_dist + 1, H]."""
    B = rel.shape[0]
    h = B // 2
    idx = []
    for n in range(int(max_dist) + 1):
        if n < h or h == 0:
            idx.append(min(n, B - 1))
        elif max_dist <= h:
            idx.append(B - 1)
        else:
            idx.append(min(B - 1, h + int(math.floor(math.log(n / h) / math.log(max_dist / h) * (B - h)))))
    return rel.float()[torch.tensor(idx, dtype=torch.long, device=rel.device)].contiguous()


def qk_norm_pages(src: torch.Tensor, H: int, Dq: int, G: int, Dk: int, Dv: int, pos: torch.Tensor,
                  slots: Optional[torch.Tensor], eps: float, temp_coef: float = 0.0, temp_every: int = 0,
                  k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Unit-normed queries and keys: of projection rows src [T, >= H Dq + G Dk + G Dv] (q | k | v,
    any row stride) every query head and key head is divided by its root mean square over the head
    (sqrt(mean x^2 + eps), no weight, fp32); queries are then multiplied by the position's
    temperature 1 + temp_coef * ln(floor((pos + 1) / temp_every) + 1) (temp_every 0: none).
    Returns q [T, H Dq]; normed keys and the values go to the paged pools (K [blocks, G, BS, Dk],
    V [blocks, G, BS / 8, Dv, 8]) at `slots` (-1: nowhere).  G = 0: queries only (a layer that
    attends over another layer's pages)."""
    T = src.shape[0]
    Cq, Ck, Cv = H * Dq, G * Dk, G * Dv
    if src.dim() != 2 or src.shape[1] < Cq + Ck + Cv or pos.shape[0] != T or src.stride(1) != 1:
        raise ValueError("qk_norm_pages: operand shapes do not fit")
    if G and (k_cache is None or v_cache is None or slots is None or tuple(k_cache.shape[1:]) != (G, k_cache.shape[2], Dk)
              or tuple(v_cache.shape[1:]) != (G, k_cache.shape[2] // 8, Dv, 8)):
        raise ValueError("qk_norm_pages: pools do not fit the key / value widths")
    if not src.is_cuda:
        x = src.float()
        q = x[:, :Cq].reshape(T, H, Dq)
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps)
        if temp_every > 0:
            tau = 1.0 + temp_coef * torch.log(torch.floor((pos.float() + 1.0) / temp_every) + 1.0)
            q = q * tau.view(T, 1, 1)
        if G:
            k = x[:, Cq:Cq + Ck].reshape(T, G, Dk)
            k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps)
            _page_write_ref(k_cache, v_cache, slots, k, x[:, Cq + Ck:Cq + Ck + Cv].reshape(T, G, Dv))
        return q.reshape(T, Cq).to(src.dtype)
    f32 = src.dtype == torch.float32
    if src.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("qk_norm_pages: bf16 or fp32 rows")
    if G and (k_cache.dtype != src.dtype or v_cache.dtype != src.dtype):
        raise ValueError("qk_norm_pages: pools share the rows' dtype")
    assert pos.dtype == torch.int32 and (slots is None or (slots.dtype == torch.int32 and slots.shape[0] == T))
    q = torch.empty(T, Cq, dtype=src.dtype, device=src.device)
    _check(lib().la_qk_norm_pages(int(f32), src.data_ptr(), src.stride(0), T, H, Dq, G, Dk, Dv, pos.data_ptr(), _ptr(slots),
                                  float(eps), float(temp_coef), int(temp_every), q.data_ptr(), _ptr(k_cache), _ptr(v_cache),
                                  k_cache.shape[2] if G else 0, _stream()), "la_qk_norm_pages")
    return q


def mamba2_states(slots: int, H: int, P: int, N: int, G: int, taps: int, dtype=torch.bfloat16, device=None):
    """State pools of ops.mamba2: (convolution tails [slots, taps - 1, H P + 2 G N] of the activation
    dtype, recurrent state fp32 [slots, H, P, N], a head's N x P state stored value-column major)."""
    return (torch.zeros(slots, max(taps - 1, 0), H * P + 2 * G * N, dtype=dtype, device=device),
            torch.zeros(slots, H, P, N, dtype=torch.float32, device=device))


def mamba2(src: torch.Tensor, H: int, P: int, N: int, G: int, conv_w: torch.Tensor, conv_b: Optional[torch.Tensor],
           dt_bias: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor, norm_w: torch.Tensor, norm_groups: int,
           eps: float, pos: torch.Tensor, cu_q: torch.Tensor, sslots: torch.Tensor, conv_state: torch.Tensor,
           ssm_state: torch.Tensor, max_rows: int = 0, conv_wt: Optional[torch.Tensor] = None) -> torch.Tensor:
    """State-space mixer with a scalar decay per head (state-space duality form) over projection
    rows src [T, 2 H P + 2 G N + H] laid out [z | x | B | C | dt]:
      * x, B, C pass a depthwise causal convolution over time (conv_w [H P + 2 G N, taps] fp32, last
        tap = current token, bias conv_b, zeros before position 0) and silu;
      * dt = softplus(dt + dt_bias) (no clamp); per head h (group floor(h / (H / G))):
        S <- exp(-exp(a_log[h]) dt) S + dt B x^T (N x P),  y = S^T C + d_skip[h] x;
      * y times silu(z), then divided by the root mean square of each of `norm_groups` equal parts
        of the H P channels (eps), times norm_w.
    Rows of a sequence portion are consecutive (cu_q [nseq + 1], pos [T]); the portion's history
    comes from conv_state[sslots[seq]] (the last taps - 1 rows of [x | B | C] before the
    convolution) and ssm_state[sslots[seq]] (fp32), both taken as zero before position 0, and both
    are advanced to the portion's end.  dt, decays, the recurrence, its state and outputs, the gate
    and the norm are fp32.  conv_wt: conv_w tap-major ([taps, C] fp32), which the vectorised
    kernel reads (widths that are multiples of 8); made per call when not given.  Returns
    [T, H P] in src's dtype."""
    T = src.shape[0]
    nseq = cu_q.shape[0] - 1
    inner, GN = H * P, G * N
    C = inner + 2 * GN
    taps = conv_w.shape[1]
    if (src.dim() != 2 or src.shape[1] != 2 * inner + 2 * GN + H or H % G or inner % norm_groups or conv_w.shape[0] != C
            or tuple(conv_state.shape[1:]) != (max(taps - 1, 0), C) or tuple(ssm_state.shape[1:]) != (H, P, N)
            or dt_bias.numel() != H or a_log.numel() != H or d_skip.numel() != H or norm_w.numel() != inner
            or sslots.shape[0] != nseq or pos.shape[0] != T or (conv_b is not None and conv_b.numel() != C)):
        raise ValueError("mamba2: operand shapes do not fit")
    if not src.is_cuda:
        u = src.float()
        z, xbc, dt = u[:, :inner], u[:, inner:inner + C], u[:, inner + C:]
        dt = torch.nn.functional.softplus(dt + dt_bias.float(), threshold=1e9)
        dec = torch.exp(-torch.exp(a_log.float()) * dt)                       # [T, H]
        y = torch.zeros(T, H, P)
        cu = cu_q.tolist()
        rep = H // G
        for s in range(nseq):
            a, b = cu[s], cu[s + 1]
            if b <= a:
                continue
            ss, p0 = int(sslots[s]), int(pos[a])
            hist = torch.zeros(taps - 1, C)
            if taps > 1:
                hist = conv_state[ss].float().clone()
                for i in range(taps - 1):            # state row i holds position p0 - (taps - 1) + i
                    if p0 - (taps - 1) + i < 0:
                        hist[i] = 0
            ext = torch.cat([hist, xbc[a:b]], 0)
            c = torch.zeros(b - a, C) if conv_b is None else conv_b.float().repeat(b - a, 1)
            for j in range(taps):
                c = c + conv_w[:, j].float() * ext[j:j + (b - a)]
            c = torch.nn.functional.silu(c)
            if taps > 1:
                conv_state[ss] = ext[-(taps - 1):].to(conv_state.dtype)
            xs = c[:, :inner].reshape(-1, H, P)
            Bm = c[:, inner:inner + GN].reshape(-1, G, N).repeat_interleave(rep, 1)
            Cm = c[:, inner + GN:].reshape(-1, G, N).repeat_interleave(rep, 1)
            S = torch.zeros(H, P, N) if p0 == 0 else ssm_state[ss].float().clone()
            for t in range(b - a):
                S = dec[a + t].view(H, 1, 1) * S + (dt[a + t].view(H, 1) * xs[t]).unsqueeze(2) * Bm[t].unsqueeze(1)
                y[a + t] = torch.einsum("hpn,hn->hp", S, Cm[t]) + d_skip.float().view(H, 1) * xs[t]
            ssm_state[ss] = S
        yg = (y.reshape(T, inner) * torch.nn.functional.silu(z)).reshape(T, norm_groups, inner // norm_groups)
        yg = yg * torch.rsqrt(yg.pow(2).mean(-1, keepdim=True) + eps)
        return (yg.reshape(T, inner) * norm_w.float()).to(src.dtype)
    f32 = src.dtype == torch.float32
    if src.dtype not in (torch.float32, torch.bfloat16) or not src.is_contiguous() or conv_state.dtype != src.dtype:
        raise ValueError("mamba2: contiguous bf16 or fp32 rows, convolution tails of the same dtype")
    if ssm_state.dtype != torch.float32 or not ssm_state.is_contiguous() or not conv_state.is_contiguous():
        raise ValueError("mamba2: the recurrent state pool is contiguous fp32")
    for t in (pos, cu_q, sslots):
        assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous()
    for t in (conv_w, conv_b, dt_bias, a_log, d_skip, norm_w):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda)
    dev = src.device
    if conv_wt is None and not (inner % 8 or GN % 8 or H % 8):
        conv_wt = conv_w.t().contiguous()
    if conv_wt is not None and (conv_wt.dtype != torch.float32 or tuple(conv_wt.shape) != (taps, C) or not conv_wt.is_contiguous()):
        raise ValueError("mamba2: conv_wt must be the fp32 [taps, C] transpose of conv_w")
    xs = torch.empty(T, inner, dtype=torch.float32, device=dev)         # convolved x
    cb = torch.empty(T, 2 * GN, dtype=torch.float32, device=dev)        # convolved C | B: the scan's q | k rows
    dtd = torch.empty(T, 2 * H, dtype=torch.float32, device=dev)        # dt | decay per (token, head)
    o = torch.empty(T, inner, dtype=torch.float32, device=dev)
    out = torch.empty(T, inner, dtype=src.dtype, device=dev)
    max_rows = int(max_rows) if max_rows > 0 else T
    seg = torch.empty((T // RETENTION_SEG + nseq) * H * P * N, dtype=torch.float32, device=dev) \
        if (T >= 8 * RETENTION_SEG and max_rows >= 4 * RETENTION_SEG) else None
    _check(lib().la_mamba2(int(f32), src.data_ptr(), T, nseq, H, P, N, G, taps, ssm_state.shape[0], conv_w.data_ptr(),
                           _ptr(conv_wt), _ptr(conv_b), dt_bias.data_ptr(), a_log.data_ptr(), d_skip.data_ptr(), norm_w.data_ptr(),
                           int(norm_groups), float(eps), pos.data_ptr(), cu_q.data_ptr(), sslots.data_ptr(),
                           conv_state.data_ptr(), ssm_state.data_ptr(), int(T == nseq and max_rows == 1), xs.data_ptr(), cb.data_ptr(),
                           dtd.data_ptr(), o.data_ptr(), out.data_ptr(), _ptr(seg), max_rows, _stream()), "la_mamba2")
    return out


# ---------------------------------------------------------------------------------------
# Layer-list designs: grouped input norms, polynomial activations, normed rotated pages with
# rotated values, the gated delta rule with a decay per key channel, stabilised matrix memories
# ---------------------------------------------------------------------------------------

def _group_rms_ref(x: torch.Tensor, w: torch.Tensor, eps: float, groups: int) -> torch.Tensor:
    T, D = x.shape
    g = x.reshape(T, groups, D // groups)
    return (g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, D) * w.float()


def add_group_norm(res: torch.Tensor, branch, w: torch.Tensor, eps: float, groups: int = 1,
                   out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Sublayer boundary of a pre-normed fp32 residual stream (fp32 [T, D], updated in place):
    res <- res + branch (a Partial or dense [T, D] tensor; None: the stream is only read), then
    returns the stream normed in `groups` equal consecutive parts, each divided by its own
    sqrt(mean(part^2) + eps), the whole times w (fp32 [D]).  All arithmetic fp32."""
    T, D = res.shape
    if groups < 1 or D % groups or w.numel() != D:
        raise ValueError("add_group_norm: the width is a multiple of the group count, w is [D]")
    if not res.is_cuda:
        if branch is not None:
            res += _branch_dense(branch)
        return _group_rms_ref(res, w, eps, groups).to(out_dtype)
    if res.dtype != torch.float32 or not res.is_contiguous() or out_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("add_group_norm: the stream is contiguous fp32; outputs are bf16 or fp32")
    if w.dtype != torch.float32 or not w.is_contiguous():
        raise ValueError("add_group_norm: weights are contiguous fp32 [D]")
    a = _branch_args(branch, T, D) if branch is not None else (None, 0, 0, 0)
    out = torch.empty(T, D, dtype=out_dtype, device=res.device)
    _check(lib().la_add_group_norm(res.data_ptr(), T, D, a[0], a[1], a[2], a[3], w.data_ptr(), float(eps), int(groups),
                                   out.data_ptr(), int(out_dtype == torch.float32), _stream()), "la_add_group_norm")
    return out


def poly_norm_act(src, coef: torch.Tensor, eps: float, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Polynomial activation with unit powers on a projection z [T, F]:  y = a N(z) + b N(z^2) + c
    N(z^3) + e, powers element by element, N(u) = u / sqrt(mean_F(u^2) + eps) over the row, (a, b,
    c, e) = coef (fp32 [4], on z's device).  fp32 arithmetic, [T, F] in out_dtype."""
    t = src.t if isinstance(src, Partial) else src
    T, F = t.shape[-2], t.shape[-1]
    if coef.numel() != 4:
        raise ValueError("poly_norm_act: four coefficients")
    if not t.is_cuda:
        z = _branch_dense(src)
        cf = coef.float()
        n = lambda u: u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)  # noqa: E731
        return (cf[0] * n(z) + cf[1] * n(z * z) + cf[2] * n(z * z * z) + cf[3]).to(out_dtype)
    if coef.dtype != torch.float32 or not coef.is_cuda:
        raise ValueError("poly_norm_act: coefficients are fp32 on the device")
    a = _branch_args(src, T, F)
    out = torch.empty(T, F, dtype=out_dtype, device=t.device)
    _check(lib().la_poly_norm_act(a[0], a[1], a[2], a[3], T, F, coef.data_ptr(), float(eps), out.data_ptr(),
                                  int(out_dtype == torch.float32), _stream()), "la_poly_norm_act")
    return out


def sigmoid_mul(x: torch.Tensor, gate: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """x * sigmoid(gate), element by element: x [T, N] contiguous, gate a [T, N] view with unit
    column stride (the gate columns of a wider projection); fp32 arithmetic."""
    T, N = x.shape
    out_dtype = out_dtype or x.dtype
    if tuple(gate.shape) != (T, N) or gate.stride(1) != 1:
        raise ValueError("sigmoid_mul: the gate is a [T, N] view with unit column stride")
    if not x.is_cuda:
        return (x.float() * torch.sigmoid(gate.float())).to(out_dtype)
    if (x.dtype not in (torch.float32, torch.bfloat16) or gate.dtype not in (torch.float32, torch.bfloat16)
            or not x.is_contiguous() or out_dtype not in (torch.float32, torch.bfloat16)):
        raise ValueError("sigmoid_mul: bf16 or fp32 operands, x contiguous")
    out = torch.empty(T, N, dtype=out_dtype, device=x.device)
    _check(lib().la_sigmoid_mul(x.data_ptr(), int(x.dtype == torch.float32), gate.data_ptr(),
                                int(gate.dtype == torch.float32), gate.stride(0), T, N, out.data_ptr(),
                                int(out_dtype == torch.float32), _stream()), "la_sigmoid_mul")
    return out


def linear_rot_freqs(dims: int, base: float, factor: float = 1.0, device=None) -> torch.Tensor:
    """Angular frequencies fp32 [dims / 2] of a rotation whose positions are divided by `factor`
    (linear position scaling): f_i = base^(-2i / dims) / factor; float64 on the host."""
    f = np.power(float(base), -2.0 * np.arange(dims // 2, dtype=np.float64) / dims) / float(factor)
    return torch.from_numpy(f.astype(np.float32)).to(device)


def qk_norm_rope_pages(src: torch.Tensor, H: int, D: int, G: int, Dv: int, pos: torch.Tensor, slots: torch.Tensor,
                       q_w: torch.Tensor, k_w: torch.Tensor, eps: float, freqs: torch.Tensor, mag: float, rot: int,
                       v_freqs: Optional[torch.Tensor], k_cache: torch.Tensor, v_cache: torch.Tensor) -> torch.Tensor:
    """Normed, rotated queries and keys and rotated values: of projection rows src [T, >= H D + G D
    + G Dv] (q | k | v, any row stride) every query and key head is divided by sqrt(mean x^2 + eps)
    and multiplied by q_w / k_w (fp32 [D], shared by the heads); then dims i and i + rot / 2 of its
    first `rot` dims are turned by the angle pos * freqs[i] (cos, sin times mag).  With v_freqs
    (fp32 [Dv / 2]) every value head is turned the same way over its whole width, dims m and m + Dv
    / 2 by pos * v_freqs[m], so that the cache holds values in the frame of their own position (an
    attention output is turned back by its query's position: rotate_heads).  Returns q [T, H D];
    keys and values go to the paged pools (K [blocks, G, BS, D], V [blocks, G, BS / 8, Dv, 8]) at
    `slots` (-1: nowhere).  Norms, angles and rotations fp32."""
    T = src.shape[0]
    Cq, Ck, Cv = H * D, G * D, G * Dv
    if (src.dim() != 2 or src.shape[1] < Cq + Ck + Cv or pos.shape[0] != T or src.stride(1) != 1 or rot % 2 or rot > D
            or freqs.numel() != rot // 2 or q_w.numel() != D or k_w.numel() != D or slots.shape[0] != T
            or (v_freqs is not None and (Dv % 2 or v_freqs.numel() != Dv // 2))):
        raise ValueError("qk_norm_rope_pages: operand shapes do not fit")
    if (tuple(k_cache.shape[1:]) != (G, k_cache.shape[2], D)
            or tuple(v_cache.shape[1:]) != (G, k_cache.shape[2] // 8, Dv, 8)):
        raise ValueError("qk_norm_rope_pages: pools do not fit the key / value widths")
    if not src.is_cuda:
        x = src.float()
        nrm = lambda y, w: y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps) * w.float()  # noqa: E731
        q = _rotate_ref(nrm(x[:, :Cq].reshape(T, H, D), q_w), pos, freqs, mag, rot, 0, False)
        k = _rotate_ref(nrm(x[:, Cq:Cq + Ck].reshape(T, G, D), k_w), pos, freqs, mag, rot, 0, False)
        v = x[:, Cq + Ck:Cq + Ck + Cv].reshape(T, G, Dv)
        if v_freqs is not None:
            v = _rotate_ref(v, pos, v_freqs, 1.0, Dv, 0, False)
        _page_write_ref(k_cache, v_cache, slots, k, v)
        return q.reshape(T, Cq).to(src.dtype)
    if src.dtype not in (torch.float32, torch.bfloat16) or k_cache.dtype != src.dtype or v_cache.dtype != src.dtype:
        raise ValueError("qk_norm_rope_pages: bf16 or fp32 rows, pools of the same dtype")
    assert pos.dtype == torch.int32 and slots.dtype == torch.int32
    for t in (q_w, k_w, freqs, v_freqs):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda)
    q = torch.empty(T, Cq, dtype=src.dtype, device=src.device)
    _check(lib().la_qk_norm_rope_pages(int(src.dtype == torch.float32), src.data_ptr(), src.stride(0), T, H, D, G, Dv,
                                       pos.data_ptr(), slots.data_ptr(), q_w.data_ptr(), k_w.data_ptr(), float(eps),
                                       _ptr(freqs) if rot else None, float(mag), rot, _ptr(v_freqs), q.data_ptr(), k_cache.data_ptr(),
                                       v_cache.data_ptr(), k_cache.shape[2], _stream()), "la_qk_norm_rope_pages")
    return q


def rotate_heads(x: torch.Tensor, H: int, Dv: int, pos: torch.Tensor, freqs: torch.Tensor, sign: float = -1.0,
                 scale: float = 1.0, out: Optional[torch.Tensor] = None, col0: int = 0) -> torch.Tensor:
    """Every head of x [T, H Dv] turned over its whole width, dims m and m + Dv / 2 by the angle
    sign * pos * freqs[m] (fp32), times `scale`; written to out[:, col0 : col0 + H Dv] (a new [T, H
    Dv] tensor of x's dtype when out is None).  sign -1 takes an attention output over values
    cached in the frame of their own positions back to the frame of its query."""
    T = x.shape[0]
    N = H * Dv
    if x.dim() != 2 or x.shape[1] != N or Dv % 2 or freqs.numel() != Dv // 2 or pos.shape[0] != T:
        raise ValueError("rotate_heads: operand shapes do not fit")
    if out is None:
        out, col0 = torch.empty(T, N, dtype=x.dtype, device=x.device), 0
    if out.shape[0] != T or col0 < 0 or col0 + N > out.shape[1] or out.stride(1) != 1 or out.dtype != x.dtype:
        raise ValueError("rotate_heads: the output window does not fit")
    if not x.is_cuda:
        y = _rotate_ref(x.float().reshape(T, H, Dv), pos.float() * sign, freqs, 1.0, Dv, 0, False) * scale
        out[:, col0:col0 + N] = y.reshape(T, N).to(out.dtype)
        return out
    if x.dtype not in (torch.float32, torch.bfloat16) or not x.is_contiguous():
        raise ValueError("rotate_heads: contiguous bf16 or fp32 rows")
    assert pos.dtype == torch.int32 and freqs.dtype == torch.float32 and freqs.is_contiguous()
    es = x.element_size()
    _check(lib().la_rotate_heads(int(x.dtype == torch.float32), x.data_ptr(), T, H, Dv, pos.data_ptr(), freqs.data_ptr(),
                                 float(sign), float(scale), out.data_ptr() + col0 * es, out.stride(0), _stream()),
           "la_rotate_heads")
    return out


def _conv_hist_ref(state, ss, p0, taps, C):
    """The taps - 1 rows before a portion that starts at position p0: the slot's tail, zeros before position 0."""
    hist = torch.zeros(max(taps - 1, 0), C)
    if taps > 1:
        hist = state[ss].float().clone()
        for i in range(taps - 1):            # state row i holds position p0 - (taps - 1) + i
            if p0 - (taps - 1) + i < 0:
                hist[i] = 0
    return hist


def delta_rule_states(slots: int, H: int, G: int, Dk: int, Dv: int, taps: int, dtype=torch.bfloat16, device=None):
    """State pools of ops.delta_rule: (convolution tails [slots, taps - 1, 2 G Dk + H Dv] of the
    activation dtype, recurrent state fp32 [slots, H, Dv, Dk], value-column major)."""
    return (torch.zeros(slots, max(taps - 1, 0), 2 * G * Dk + H * Dv, dtype=dtype, device=device),
            torch.zeros(slots, H, Dv, Dk, dtype=torch.float32, device=device))


def delta_rule(src: torch.Tensor, dec: torch.Tensor, gate: torch.Tensor, H: int, G: int, Dk: int, Dv: int,
               conv_w: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, norm_w: torch.Tensor, eps: float,
               pos: torch.Tensor, cu_q: torch.Tensor, sslots: torch.Tensor, conv_state: torch.Tensor,
               rec_state: torch.Tensor, unit_eps: float = 1e-6, max_rows: int = 0,
               conv_wt: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Gated delta rule with one decay per head and key channel over projection rows src [T, >= 2 G
    Dk + H Dv + H] laid out [q | k | v | beta logits] (any row stride), dec [T, H Dk] (decay
    logits) and gate [T, H Dv] (output gate logits):
      * q, k (G heads of width Dk; head h reads group floor(h / (H / G))) and v (H heads of width
        Dv) pass a depthwise causal convolution over time (conv_w [2 G Dk + H Dv, taps] fp32, last
        tap = current token, no bias, zeros before position 0) and silu;
      * q and k become unit vectors per head, x / sqrt(sum x^2 + unit_eps); q times Dk^-1/2;
      * beta = sigmoid(beta logits); g = exp(-exp(a_log[h]) softplus(dec + dt_bias)) per (head, key channel);
      * per head, S (Dk x Dv):  S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;
      * o divided by its root mean square over the head's Dv (eps), times norm_w (fp32 [Dv], shared
        by the heads), times sigmoid(gate).
    Rows of a sequence portion are consecutive (cu_q [nseq + 1], pos [T]); the portion's history
    comes from conv_state[sslots[seq]] (the last taps - 1 rows of [q | k | v] before the
    convolution) and rec_state[sslots[seq]] (fp32 [H, Dv, Dk]), both taken as zero before position
    0, and both are advanced to the portion's end.  Everything after the convolution's silu is
    fp32.  conv_wt: conv_w tap-major ([taps, C] fp32), which the vectorised bf16 kernel reads (key and
    value widths and the row stride multiples of 8); made per call when not given.  Returns [T, H Dv]
    in src's dtype."""
    T = src.shape[0]
    nseq = cu_q.shape[0] - 1
    Cqk, Cv = G * Dk, H * Dv
    C = 2 * Cqk + Cv
    taps = conv_w.shape[1]
    if (src.dim() != 2 or src.shape[1] < C + H or src.stride(1) != 1 or H % G or conv_w.shape[0] != C
            or tuple(dec.shape) != (T, H * Dk) or tuple(gate.shape) != (T, Cv)
            or tuple(conv_state.shape[1:]) != (max(taps - 1, 0), C) or tuple(rec_state.shape[1:]) != (H, Dv, Dk)
            or dt_bias.numel() != H * Dk or a_log.numel() != H or norm_w.numel() != Dv or sslots.shape[0] != nseq
            or pos.shape[0] != T):
        raise ValueError("delta_rule: operand shapes do not fit")
    if not src.is_cuda:
        u_ = src[:, :C].float()
        beta = torch.sigmoid(src[:, C:C + H].float())
        dt = torch.nn.functional.softplus(dec.float() + dt_bias.float(), threshold=1e9).view(T, H, Dk)
        gdec = torch.exp(-torch.exp(a_log.float()).view(1, H, 1) * dt)
        o = torch.zeros(T, H, Dv)
        cu = cu_q.tolist()
        rep = H // G
        for s in range(nseq):
            a, b = cu[s], cu[s + 1]
            if b <= a:
                continue
            ss, p0 = int(sslots[s]), int(pos[a])
            ext = torch.cat([_conv_hist_ref(conv_state, ss, p0, taps, C), u_[a:b]], 0)
            c = torch.zeros(b - a, C)
            for j in range(taps):
                c = c + conv_w[:, j].float() * ext[j:j + (b - a)]
            c = torch.nn.functional.silu(c)
            if taps > 1:
                conv_state[ss] = ext[-(taps - 1):].to(conv_state.dtype)
            q = c[:, :Cqk].reshape(-1, G, Dk)
            k = c[:, Cqk:2 * Cqk].reshape(-1, G, Dk)
            q = (q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + unit_eps) * Dk ** -0.5).repeat_interleave(rep, 1)
            k = (k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + unit_eps)).repeat_interleave(rep, 1)
            v = c[:, 2 * Cqk:].reshape(-1, H, Dv)
            S = torch.zeros(H, Dk, Dv) if p0 == 0 else rec_state[ss].float().transpose(1, 2).clone()
            for t in range(b - a):
                S = gdec[a + t].unsqueeze(2) * S
                uu = beta[a + t].view(H, 1) * (v[t] - torch.einsum("hkv,hk->hv", S, k[t]))
                S = S + k[t].unsqueeze(2) * uu.unsqueeze(1)
                o[a + t] = torch.einsum("hkv,hk->hv", S, q[t])
            rec_state[ss] = S.transpose(1, 2)
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
        return (o.reshape(T, Cv) * torch.sigmoid(gate.float())).to(src.dtype)
    f32 = src.dtype == torch.float32
    if src.dtype not in (torch.float32, torch.bfloat16) or conv_state.dtype != src.dtype or dec.dtype != src.dtype \
            or gate.dtype != src.dtype or not dec.is_contiguous() or not gate.is_contiguous():
        raise ValueError("delta_rule: bf16 or fp32 rows; tails, decay and gate logits of the same dtype")
    if rec_state.dtype != torch.float32 or not rec_state.is_contiguous() or not conv_state.is_contiguous():
        raise ValueError("delta_rule: the recurrent state pool is contiguous fp32")
    for t in (pos, cu_q, sslots):
        assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous()
    for t in (conv_w, dt_bias, a_log, norm_w):
        assert t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda
    dev = src.device
    if conv_wt is None and not f32 and not (Dk % 8 or Dv % 8 or src.stride(0) % 8):
        conv_wt = conv_w.t().contiguous()
    if conv_wt is not None and (conv_wt.dtype != torch.float32 or tuple(conv_wt.shape) != (taps, C) or not conv_wt.is_contiguous()):
        raise ValueError("delta_rule: conv_wt must be the fp32 [taps, C] transpose of conv_w")
    qk = torch.empty(T, 2 * Cqk, dtype=torch.float32, device=dev)       # unit q (scaled) | unit k per group
    vf = torch.empty(T, Cv, dtype=torch.float32, device=dev)            # convolved v
    gd = torch.empty(T, H * Dk, dtype=torch.float32, device=dev)        # decays per (token, head, key channel)
    bq = torch.empty(T, H + G, dtype=torch.float32, device=dev)         # beta per head | k . q per group
    o = torch.empty(T, Cv, dtype=torch.float32, device=dev)
    out = torch.empty(T, Cv, dtype=src.dtype, device=dev)
    max_rows = int(max_rows) if max_rows > 0 else T
    _check(lib().la_delta_rule(int(f32), src.data_ptr(), src.stride(0), dec.data_ptr(), gate.data_ptr(), T, nseq, H, G, Dk,
                               Dv, taps, rec_state.shape[0], conv_w.data_ptr(), _ptr(conv_wt), dt_bias.data_ptr(), a_log.data_ptr(),
                               norm_w.data_ptr(), float(eps), float(unit_eps), pos.data_ptr(), cu_q.data_ptr(),
                               sslots.data_ptr(), conv_state.data_ptr(), rec_state.data_ptr(),
                               int(T == nseq and max_rows == 1), qk.data_ptr(), vf.data_ptr(), gd.data_ptr(), bq.data_ptr(),
                               o.data_ptr(), out.data_ptr(), _stream()), "la_delta_rule")
    return out


def matrix_memory_states(slots: int, H: int, Dk: int, Dv: int, device=None):
    """State pools of ops.matrix_memory: (fp32 [slots, H, Dv + 1, Dk]: the Dk x Dv memory
    value-column major with the normaliser vector as one more column, fp32 [slots, H]: the running
    maximum of the gates' logarithms)."""
    return (torch.zeros(slots, H, Dv + 1, Dk, dtype=torch.float32, device=device),
            torch.zeros(slots, H, dtype=torch.float32, device=device))


def matrix_memory(src: torch.Tensor, H: int, Dk: int, Dv: int, gate_b: torch.Tensor, cap: float, norm_w: torch.Tensor,
                  eps: float, pos: torch.Tensor, cu_q: torch.Tensor, sslots: torch.Tensor, mem_state: torch.Tensor,
                  max_state: torch.Tensor, scale: float = 1.0, denom_eps: float = 1e-6, max_rows: int = 0,
                  out: Optional[torch.Tensor] = None, col0: int = 0) -> torch.Tensor:
    """Matrix memory with exponential gates kept in range by a running maximum, over projection
    rows src [T, >= 2 H Dk + 2 H Dv + 2 H] laid out [q | k | v | output gate | input gate | forget
    gate] (any row stride); gate_b fp32 [2 H]: the input and forget gates' biases.  Per head:
      i = cap tanh((input + b) / cap),  f = logsigmoid(cap tanh((forget + b) / cap)),  q times Dk^-1/2;
      m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k alone;
      o = S^T q / (max(|n . q|, exp(-m')) + denom_eps);
    o divided by its root mean square over the head's Dv (eps), times norm_w (fp32 [H Dv]), times
    sigmoid(output gate), times `scale`.  S, n and m of a sequence live in mem_state[sslots[seq]]
    (fp32 [H, Dv + 1, Dk], n as the last column) and max_state[sslots[seq]] (fp32 [H]); all start at
    zero at position 0 (m too) and are advanced to the portion's end.  Gates, the recurrence and the
    norm are fp32.  Written to out[:, col0 : col0 + H Dv] (a new tensor of src's dtype when None)."""
    T = src.shape[0]
    nseq = cu_q.shape[0] - 1
    Cq, Cv = H * Dk, H * Dv
    W = 2 * Cq + 2 * Cv + 2 * H
    if (src.dim() != 2 or src.shape[1] < W or src.stride(1) != 1 or tuple(mem_state.shape[1:]) != (H, Dv + 1, Dk)
            or tuple(max_state.shape[1:]) != (H,) or gate_b.numel() != 2 * H or norm_w.numel() != Cv
            or sslots.shape[0] != nseq or pos.shape[0] != T):
        raise ValueError("matrix_memory: operand shapes do not fit")
    if out is None:
        out, col0 = torch.empty(T, Cv, dtype=src.dtype, device=src.device), 0
    if out.shape[0] != T or col0 < 0 or col0 + Cv > out.shape[1] or out.stride(1) != 1 or out.dtype != src.dtype:
        raise ValueError("matrix_memory: the output window does not fit")
    if not src.is_cuda:
        x = src.float()
        q = x[:, :Cq].reshape(T, H, Dk) * Dk ** -0.5
        k = x[:, Cq:2 * Cq].reshape(T, H, Dk)
        v = x[:, 2 * Cq:2 * Cq + Cv].reshape(T, H, Dv)
        og = x[:, 2 * Cq + Cv:2 * Cq + 2 * Cv]
        b = gate_b.float()
        ig = cap * torch.tanh((x[:, W - 2 * H:W - H] + b[:H]) / cap)
        fg = torch.nn.functional.logsigmoid(cap * torch.tanh((x[:, W - H:W] + b[H:]) / cap))
        o = torch.zeros(T, H, Dv)
        cu = cu_q.tolist()
        for s in range(nseq):
            a, e = cu[s], cu[s + 1]
            if e <= a:
                continue
            ss = int(sslots[s])
            if int(pos[a]) == 0:
                S, n, m = torch.zeros(H, Dk, Dv), torch.zeros(H, Dk), torch.zeros(H)
            else:
                st = mem_state[ss].float()
                S, n, m = st[:, :Dv].transpose(1, 2).clone(), st[:, Dv].clone(), max_state[ss].float().clone()
            for t in range(a, e):
                m2 = torch.maximum(fg[t] + m, ig[t])
                fa, ia = torch.exp(fg[t] + m - m2), torch.exp(ig[t] - m2)
                S = fa.view(H, 1, 1) * S + ia.view(H, 1, 1) * k[t].unsqueeze(2) * v[t].unsqueeze(1)
                n = fa.view(H, 1) * n + ia.view(H, 1) * k[t]
                m = m2
                den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + denom_eps
                o[t] = torch.einsum("hkv,hk->hv", S, q[t]) / den.view(H, 1)
            mem_state[ss, :, :Dv] = S.transpose(1, 2)
            mem_state[ss, :, Dv] = n
            max_state[ss] = m
        o = (o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, Cv)
        out[:, col0:col0 + Cv] = (o * norm_w.float() * torch.sigmoid(og) * scale).to(out.dtype)
        return out
    f32 = src.dtype == torch.float32
    if src.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("matrix_memory: bf16 or fp32 rows")
    if (mem_state.dtype != torch.float32 or max_state.dtype != torch.float32 or not mem_state.is_contiguous()
            or not max_state.is_contiguous()):
        raise ValueError("matrix_memory: the state pools are contiguous fp32")
    for t in (pos, cu_q, sslots):
        assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous()
    for t in (gate_b, norm_w):
        assert t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda
    dev = src.device
    Dv1 = Dv + 1
    qk = torch.empty(T, 2 * Cq, dtype=torch.float32, device=dev)       # scaled q | k
    va = torch.empty(T, H * Dv1, dtype=torch.float32, device=dev)      # v with a column of ones per head
    gts = torch.empty(T, 3 * H, dtype=torch.float32, device=dev)       # decay | input scale | exp(-m) per (token, head)
    o = torch.empty(T, H * Dv1, dtype=torch.float32, device=dev)
    max_rows = int(max_rows) if max_rows > 0 else T
    seg = torch.empty((T // RETENTION_SEG + nseq) * H * Dv1 * Dk, dtype=torch.float32, device=dev) \
        if (T >= 8 * RETENTION_SEG and max_rows >= 4 * RETENTION_SEG) else None
    es = src.element_size()
    _check(lib().la_matrix_memory(int(f32), src.data_ptr(), src.stride(0), T, nseq, H, Dk, Dv, gate_b.data_ptr(), float(cap),
                                  norm_w.data_ptr(), float(eps), float(denom_eps), float(scale), pos.data_ptr(),
                                  cu_q.data_ptr(), sslots.data_ptr(), mem_state.data_ptr(), max_state.data_ptr(),
                                  mem_state.shape[0], qk.data_ptr(), va.data_ptr(), gts.data_ptr(), o.data_ptr(),
                                  out.data_ptr() + col0 * es, out.stride(0), _ptr(seg), max_rows, _stream()),
           "la_matrix_memory")
    return out


# ---------------------------------------------------------------------------------------
# Sampling
# ---------------------------------------------------------------------------------------

SAMPLE_ROW_DTYPE = np.dtype([("temp", "<f4"), ("top_p", "<f4"), ("min_p", "<f4"), ("typical_p", "<f4"),
                             ("tfs_z", "<f4"), ("tau", "<f4"), ("eta", "<f4"), ("top_k", "<i4"),
                             ("mirostat", "<i4"), ("pad", "<i4"), ("seed", "<u8"), ("counter", "<u8")])


def sample(logits: torch.Tensor, params: np.ndarray, mu: Optional[torch.Tensor] = None,
           params_dev: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """logits [B, V] f32; params: structured array (SAMPLE_ROW_DTYPE) of length B."""
    B, V = logits.shape
    assert params.dtype == SAMPLE_ROW_DTYPE and len(params) == B
    if not logits.is_cuda:
        return sample_ref(logits, params, mu)
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise ValueError("sample: logits must be f32 with unit column stride")
    if params_dev is None:
        params_dev = torch.from_numpy(params.view(np.uint8).copy()).to(logits.device, non_blocking=True)
    if mu is None:
        mu = torch.zeros(B, dtype=torch.float32, device=logits.device)
    if out is None:
        out = torch.empty(B, dtype=torch.int32, device=logits.device)
    _check(lib().la_sample(logits.data_ptr(), logits.stride(0), B, V, params_dev.data_ptr(), mu.data_ptr(),
                           out.data_ptr(), None, _stream()), "la_sample")
    return out


def sample_ref(logits: torch.Tensor, params: np.ndarray, mu: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Host reference of the sampler chain (same semantics, torch RNG)."""
    B, V = logits.shape
    out = torch.empty(B, dtype=torch.int32)
    for b in range(B):
        p = params[b]
        l = logits[b].float().cpu()
        if p["temp"] <= 0:
            out[b] = int(torch.argmax(l))
            continue
        g = torch.Generator().manual_seed(int(p["seed"]) ^ int(p["counter"]))
        if p["mirostat"] == 2:
            pr = torch.softmax(l / float(p["temp"]), -1)
            m = float(mu[b]) if mu is not None else 2 * float(p["tau"])
            keep = pr >= 2.0 ** (-m)
            keep[torch.argmax(pr)] = True
            q = torch.where(keep, pr, torch.zeros_like(pr))
            q = q / q.sum()
            t = int(torch.multinomial(q, 1, generator=g))
            if mu is not None:
                mu[b] = m - float(p["eta"]) * (-math.log2(float(q[t])) - float(p["tau"]))
            out[b] = t
            continue
        vals, idx = torch.sort(l, descending=True, stable=True)
        k = int(p["top_k"])
        if 0 < k < V:
            vals, idx = vals[:k], idx[:k]
        pr = torch.softmax(vals, -1)
        n = len(vals)
        if p["top_p"] < 1:
            cs = torch.cumsum(pr, 0)
            hit = torch.nonzero(cs >= float(p["top_p"]))
            if len(hit):
                n = min(n, int(hit[0]) + 1)
        if p["min_p"] > 0:
            keepm = int((vals >= vals[0] + math.log(float(p["min_p"]))).sum())
            n = min(n, max(1, keepm))
        vals, idx = vals[:n], idx[:n]
        q = torch.softmax(vals / float(p["temp"]), -1)
        out[b] = int(idx[int(torch.multinomial(q, 1, generator=g))])
    return out


def logit_bias(logits: torch.Tensor, rows: torch.Tensor, cols: torch.Tensor, vals: torch.Tensor,
               count: torch.Tensor):
    """In place: logits[rows[i], cols[i]] += vals[i] for i < count[0] (graph-capturable: the
    entry count lives on the device)."""
    cap = rows.shape[0]
    if not logits.is_cuda:
        n = int(count[0])
        logits.index_put_((rows[:n].long(), cols[:n].long()), vals[:n].to(logits.dtype), accumulate=True)
        return logits
    _check(lib().la_logit_bias(logits.data_ptr(), logits.stride(0), rows.data_ptr(), cols.data_ptr(),
                               vals.data_ptr(), count.data_ptr(), cap, _stream()), "la_logit_bias")
    return logits


def decode_advance(next_tok, tok, pos, lens, slots, bt, block_size: int, hist, step, prm_dev):
    """Feed sampled tokens back as the next decode inputs (see csrc/decode_loop.hip)."""
    B = tok.shape[0]
    if not tok.is_cuda:
        s = int(step[0])
        if s < hist.shape[0]:
            hist[s] = next_tok
        live = slots >= 0
        tok[live] = next_tok[live]
        pos[live] += 1
        lens[live] = pos[live] + 1
        p = pos[live].long()
        slots[live] = (bt[live, p // block_size] * block_size + (p % block_size)).to(slots.dtype)
        rows = prm_dev.numpy().view(SAMPLE_ROW_DTYPE)
        rows["counter"][live.numpy()] += 1
        step[0] = s + 1
        return
    _check(lib().la_decode_advance(next_tok.data_ptr(), tok.data_ptr(), pos.data_ptr(), lens.data_ptr(),
                                   slots.data_ptr(), bt.data_ptr(), bt.stride(0), block_size, B, hist.data_ptr(),
                                   hist.shape[0], step.data_ptr(), prm_dev.data_ptr(), _stream()),
           "la_decode_advance")


# ---------------------------------------------------------------------------------------
# Mixture of experts (decode-sized batches; csrc/moe.hip)
# ---------------------------------------------------------------------------------------

class MoEWeights:
    """E experts of one projection (same format / shape) + their QW descriptors on the device."""

    def __init__(self, experts: Sequence[QWeight]):
        if not experts or len({(w.fmt, w.N, w.K) for w in experts}) != 1:
            raise ValueError("MoEWeights: experts must share format and shape")
        self.experts = list(experts)
        self.E, self.N, self.K, self.fmt = len(experts), experts[0].N, experts[0].K, experts[0].fmt
        self.desc = None
        p0 = experts[0].planes[0]
        if p0 is not None and p0.device.type == "cuda":
            dev = p0.device
            qw = np.zeros(self.E, dtype=[("p", "<u8", 4), ("N", "<i4"), ("K", "<i4")])
            assert qw.dtype.itemsize == lib().la_qw_size()
            for e, w in enumerate(experts):
                qw[e]["p"] = [_ptr(p) or 0 for p in w.planes]
                qw[e]["N"], qw[e]["K"] = w.N, w.K
            self.desc = torch.from_numpy(qw.view(np.uint8).copy()).to(dev)
        self._desc32 = None

    def desc32(self) -> torch.Tensor:
        """Descriptors for the 32x32x16 grouped GEMM (la_moe32): {codes, aux, blocked scale
        plane, -} per expert; the scale planes are built on first use (0.125 B per weight)."""
        if self._desc32 is None:
            qw = np.zeros(self.E, dtype=[("p", "<u8", 4), ("N", "<i4"), ("K", "<i4")])
            for e, w in enumerate(self.experts):
                p0, p1, g = w.tile_planes()
                qw[e]["p"] = [p0 or 0, p1 or 0, g or 0, 0]
                qw[e]["N"], qw[e]["K"] = w.N, w.K
            self._desc32 = torch.from_numpy(qw.view(np.uint8).copy()).to(self.desc.device)
        return self._desc32


def moe_router(xn: torch.Tensor, router: torch.Tensor, topk: int, renorm: bool, scale: float = 1.0,
               ep_base: int = 0, ep_local: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    """Fused router for decode batches: xn [T, D] bf16, router [E, D] fp32 -> (ids [T, topk] int32,
    weights [T*topk] fp32): softmax over E, top-k by probability, optional renormalisation and
    scale; under expert parallelism ids are local (ep_base..ep_base+ep_local-1 -> 0..) and other
    ranks' experts map to ep_local."""
    T, D = xn.shape
    E = router.shape[0]
    local = ep_local or E
    if not xn.is_cuda:
        p = torch.softmax(xn.float() @ router.t(), -1)
        w, idx = torch.topk(p, topk, -1)
        if renorm:
            w = w / w.sum(-1, keepdim=True)
        loc = idx - ep_base
        ids = torch.where((loc >= 0) & (loc < local), loc, torch.full_like(loc, local)).to(torch.int32)
        return ids, (w * scale).reshape(-1).float()
    assert xn.dtype == torch.bfloat16 and xn.stride(-1) == 1 and router.dtype == torch.float32
    assert router.is_contiguous() and router.shape[1] == D and D % 8 == 0 and E <= 256 and topk <= min(16, E)
    ids = torch.empty(T, topk, dtype=torch.int32, device=xn.device)
    wts = torch.empty(T * topk, dtype=torch.float32, device=xn.device)
    _check(lib().la_moe_router(xn.data_ptr(), xn.stride(0), router.data_ptr(), E, D, T, topk, int(renorm),
                               float(scale), ep_base, local, ids.data_ptr(), wts.data_ptr(), _stream()),
           "la_moe_router")
    return ids, wts


def moe_route(ids: torch.Tensor, E: int, order: Optional[torch.Tensor] = None, off: Optional[torch.Tensor] = None):
    """ids [T, topk] int32 -> (order [T*topk] pair ids grouped by expert, off [E+1])."""
    T, topk = ids.shape
    if order is None:
        order = torch.empty(T * topk, dtype=torch.int32, device=ids.device)
    if off is None:
        off = torch.empty(E + 1, dtype=torch.int32, device=ids.device)
    if not ids.is_cuda:
        flat = ids.reshape(-1).long()
        perm = torch.sort(flat, stable=True).indices
        order.copy_(perm.to(torch.int32))
        cnt = torch.bincount(flat, minlength=E)
        off.copy_(torch.cat([torch.zeros(1, dtype=torch.long), cnt.cumsum(0)]).to(torch.int32))
        return order, off
    ids = ids.contiguous().to(torch.int32)
    _check(lib().la_moe_route(ids.data_ptr(), T, topk, E, order.data_ptr(), off.data_ptr(), _stream()), "la_moe_route")
    return order, off


def moe_linear(x: torch.Tensor, mw: MoEWeights, order: torch.Tensor, off: torch.Tensor, topk: int, T: int,
               down: bool = False, wts: Optional[torch.Tensor] = None, zero: bool = False) -> Partial:
    """Grouped expert GEMM.  gate/up (down=False): x [T, K] -> Partial [S, T*topk, N] (row = pair).
    down (down=True): x [T*topk, K] (row = pair) -> Partial [S*topk, T, N], each slab scaled by
    the routing weight, so summing the slabs performs the weighted top-k combine.  Pairs routed to
    an expert id >= mw.E (expert parallelism: another rank's expert) are not computed; with
    zero=True their down-projection rows read as 0."""
    if not x.is_cuda:
        P = T * topk
        flat_e = torch.full((P,), -1, dtype=torch.long)
        offs = off.tolist()
        for e in range(mw.E):
            flat_e[order[offs[e]:offs[e + 1]].long()] = e
        if down:
            out = torch.zeros(topk, T, mw.N)
            for p in range(P):
                t, slot = divmod(p, topk)
                if flat_e[p] < 0:
                    continue
                out[slot, t] = (x[p].float() @ mw.experts[int(flat_e[p])].dequant_f32().t()) * float(wts[p])
        else:
            out = torch.zeros(1, P, mw.N)
            for p in range(P):
                if flat_e[p] >= 0:
                    out[0, p] = x[p // topk].float() @ mw.experts[int(flat_e[p])].dequant_f32().t()
        return Partial(out)
    if x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("moe_linear: x must be contiguous bf16")
    maxM = T  # a token picks an expert at most once; above 64 rows the launch adds row chunks
    S = pick_splits(mw.N, mw.K, maxM)
    nsb = mw.K // 256
    while nsb % S:
        S -= 1
    P = T * topk
    if down:
        alloc = torch.zeros if zero else torch.empty
        out = alloc(S * topk, T, mw.N, dtype=torch.float32, device=x.device)
        slab = T * mw.N
    else:
        out = torch.empty(S, P, mw.N, dtype=torch.float32, device=x.device)
        slab = P * mw.N
    _check(lib().la_moe_gemm(mw.fmt, 1 if down else 0, mw.desc.data_ptr(), mw.N, mw.K, mw.E, order.data_ptr(),
                             off.data_ptr(), topk, x.data_ptr(), x.shape[1], maxM, S,
                             _ptr(wts) if down else None, out.data_ptr(), mw.N, slab, T, _stream()), "la_moe_gemm")
    return Partial(out)


# Grouped expert GEMMs on the 32x32x16 tile (gemm_q32.hip moe32_kernel) for batches of at least
# MOE32_MIN_T tokens: gate|up with the SwiGLU fused (bf16 h in grouped row order), then the
# routing-weighted down projection.  Variant ids: gemm_q32.hip moe32_var.
MOE32 = os.environ.get("LOCALAI_AMD_MOE32", "1") == "1"
# Variant by batch (scripts/moe_bench.py, Mixtral-8x7B shapes, gpurun_out/r5_moe32_bench.log):
# T = 64: 32-row tiles, 4 workgroups per CU (var 9) 156 + 86 us vs the 16-column kernel's
# 285 + 9 (act) + 143; T = 128 / 256: 64-row tiles in 8-wave workgroups (var 4) 180 + 91 /
# 291 + 162 us vs 276 + 15 + 145 / 470 + 16 + 255.
# T = 16 / 24 / 32: var 9 232 / 234 / 237 us vs 266 / 315 / 317; T = 8: 221 vs 212
# (gpurun_out/r5_moe_small.log)
MOE32_MIN_T = int(os.environ.get("LOCALAI_AMD_MOE32_MIN_T", "12"))
MOE32_SMALL_T = 48     # below: var 9 (32-row tiles); from here: var 17 (64-row chunks, live row blocks)
MOE32_LIVE_BIG_T = 192  # from here: var 19 (one 128-row chunk per expert at top-2 of 8)
MOE32_VAR_GLU = int(os.environ.get("LOCALAI_AMD_MOE32_VAR_GLU", "-1"))     # -1: by batch
MOE32_VAR_DOWN = int(os.environ.get("LOCALAI_AMD_MOE32_VAR_DOWN", "-1"))
MOE32_SPLITS = int(os.environ.get("LOCALAI_AMD_MOE32_SPLITS", "0"))   # 0: picked from the tile count
MOE32_TILES = {0: (64, 128), 1: (64, 128), 2: (64, 256), 3: (64, 256), 4: (64, 256), 5: (32, 128), 6: (128, 128),
               7: (64, 128), 8: (64, 128), 9: (32, 128), 10: (32, 256), 11: (64, 256), 12: (32, 256),
               13: (64, 128), 14: (32, 256), 15: (128, 256), 16: (128, 128), 17: (64, 256), 18: (128, 128),
               19: (128, 512), 20: (128, 256)}
_MOE32_FMTS = (FMT_Q4_K, FMT_Q6_K, FMT_Q8_0)


def moe32_ok(gu: "MoEWeights", down: "MoEWeights", T: int) -> bool:
    """Can the gate|up / down pair of a layer run on la_moe32 for a T-token batch."""
    return (MOE32 and T >= MOE32_MIN_T and gu.desc is not None and down.desc is not None
            and gu.fmt in _MOE32_FMTS and down.fmt in _MOE32_FMTS and gu.K % 256 == 0 and down.K % 256 == 0
            and gu.N % 32 == 0 and down.K == gu.N // 2)


def moe_glu32(x: torch.Tensor, mw: "MoEWeights", order: torch.Tensor, off: torch.Tensor, topk: int, T: int,
              act: int = ACT_SWIGLU, var: Optional[int] = None) -> torch.Tensor:
    """h = act(x Wg^T) * (x Wu^T) for every routed pair: x [T, K] bf16 -> h [T*topk, F] bf16 in
    the grouping's row order (row off[e] + m is pair order[off[e] + m]); rows of pairs routed to
    no local expert stay unwritten (the down projection never reads them)."""
    F = mw.N // 2
    if x.dtype != torch.bfloat16 or not x.is_contiguous() or x.shape[1] != mw.K:
        raise ValueError("moe_glu32: x must be contiguous bf16 [T, K]")
    h = torch.empty(T * topk, F, dtype=torch.bfloat16, device=x.device)
    a = {ACT_SWIGLU: 0, ACT_GEGLU: 3}[act]
    _check(lib().la_moe32(mw.fmt, 1, mw.desc32().data_ptr(), F, mw.K, mw.E, order.data_ptr(), off.data_ptr(), topk,
                          x.data_ptr(), x.shape[1], T, 1, None, h.data_ptr(), F, 0, a,
                          _moe32_var(MOE32_VAR_GLU, T, mw.fmt) if var is None else var, _stream()), "la_moe32")
    return h


def _moe32_var(env: int, T: int, fmt: int = FMT_Q4_K, down: bool = False) -> int:
    if env >= 0:
        return env
    # live-row-block variants (profiles/r6_moe_live.md, Mixtral-8x7B shapes, cold weights): T = 256
    # var 19 (128-row chunks, 8 waves x 64 columns) glu 244 + down 118 us vs var 15's 280 + 131 on
    # the same box and var 4's 315 + 170 on another; T = 64 / 128
    # var 17 (64-row chunks) 167 + 82 / 172 + 86 vs var 9's 166 + 91 / var 4's 180 + 91; below
    # MOE32_SMALL_T var 9 (32-row tiles, 4 workgroups per CU) stays for the smallest batches
    if T >= MOE32_LIVE_BIG_T:
        # var 19's 64-column waves spill with Q6_K / Q8_0 fragments (the launcher maps them to 15)
        return 19 if fmt == FMT_Q4_K else 15
    return 9 if T < MOE32_SMALL_T else 17


def _moe32_splits(mw: "MoEWeights", T: int, topk: int, var: int) -> int:
    if MOE32_SPLITS:
        S = MOE32_SPLITS
    else:
        bm, bn = MOE32_TILES[var]
        live = (-(-T * topk // bm) + mw.E // 2) * -(-mw.N // bn)   # tiles with rows (balanced router)
        S = 1
        while S < 8 and live * S * 2 <= 1024 and mw.K // 64 >= 64 * S:
            S *= 2
    ks = mw.K // 64
    while S > 1 and -(-ks // S) * (S - 1) >= ks:
        S -= 1
    return S


def moe_down32(h: torch.Tensor, mw: "MoEWeights", order: torch.Tensor, off: torch.Tensor, topk: int, T: int,
               wts: torch.Tensor, zero: bool = False, var: Optional[int] = None) -> Partial:
    """Down projection of moe_glu32's grouped h rows -> Partial [S*topk, T, N]: slab
    (split*topk + slot) row t holds wts[pair] * (h_pair Wd^T) of token t's slot-th pick, so the
    consumer's slab sum is the weighted top-k combine (moe_linear's down contract)."""
    v = _moe32_var(MOE32_VAR_DOWN, T, mw.fmt, down=True) if var is None else var
    S = _moe32_splits(mw, T, topk, v)
    alloc = torch.zeros if zero else torch.empty
    out = alloc(S * topk, T, mw.N, dtype=torch.float32, device=h.device)
    _check(lib().la_moe32(mw.fmt, 2, mw.desc32().data_ptr(), mw.N, mw.K, mw.E, order.data_ptr(), off.data_ptr(), topk,
                          h.data_ptr(), h.shape[1], T, S, wts.data_ptr(), out.data_ptr(), mw.N, T * mw.N, 0, v,
                          _stream()), "la_moe32")
    return Partial(out)


# Grouped MoE on the shared-dequant-image tile (gemm_bs.hip bsmoe_kernel): every local expert's
# routed rows in ONE launch per projection, 256-row tiles (an expert's weights stream once per 256
# rows, not once per 64 as on moe32), grid sized for any routing -- no host read of the grouping.
# Prefill chunks (T >= MOE_BS_MIN_T tokens); decode batches stay on moe32.
# opt-in: slower than both the grouped moe32 tiles and the dense per-expert path on Mixtral-8x7B
# prefill chunks (profiles/r6_moe_live.md)
MOE_BS = os.environ.get("LOCALAI_AMD_MOE_BS", "0") == "1"
MOE_BS_MIN_T = int(os.environ.get("LOCALAI_AMD_MOE_BS_MIN_T", "512"))
MOE_BS_VAR = int(os.environ.get("LOCALAI_AMD_MOE_BS_VAR", "0"))


def moe_bs_ok(gu: "MoEWeights", down: "MoEWeights", T: int) -> bool:
    """Can the gate|up / down pair of a layer run on la_bsmoe for a T-token chunk."""
    return (MOE_BS and T >= MOE_BS_MIN_T and gu.desc is not None and down.desc is not None
            and gu.fmt in _MOE32_FMTS and down.fmt in _MOE32_FMTS and gu.K % 256 == 0 and down.K % 256 == 0
            and gu.N % 16 == 0 and down.N % 4 == 0 and down.K == gu.N // 2)


def moe_glu_bs(x: torch.Tensor, mw: "MoEWeights", order: torch.Tensor, off: torch.Tensor, topk: int, T: int,
               act: int = ACT_SWIGLU, var: Optional[int] = None) -> torch.Tensor:
    """moe_glu32's contract on the bs tile: h [T*topk, F] bf16 in grouped row order."""
    F = mw.N // 2
    if x.dtype != torch.bfloat16 or not x.is_contiguous() or x.shape[1] != mw.K or x.shape[0] != T:
        raise ValueError("moe_glu_bs: x must be contiguous bf16 [T, K]")
    h = torch.empty(T * topk, F, dtype=torch.bfloat16, device=x.device)
    a = {ACT_SWIGLU: 0, ACT_GEGLU: 3}[act]
    _check(lib().la_bsmoe(mw.fmt, 1, mw.desc32().data_ptr(), F, mw.K, mw.E, order.data_ptr(), off.data_ptr(), topk,
                          x.data_ptr(), x.shape[1], T, 1, None, h.data_ptr(), F, 0, a,
                          MOE_BS_VAR if var is None else var, _stream()), "la_bsmoe")
    return h


def moe_down_bs(h: torch.Tensor, mw: "MoEWeights", order: torch.Tensor, off: torch.Tensor, topk: int, T: int,
                wts: torch.Tensor, zero: bool = False, var: Optional[int] = None) -> Partial:
    """moe_down32's contract on the bs tile: Partial [topk, T, N], slab `slot` row t = wts[pair] *
    (h_pair Wd^T) of token t's slot-th pick."""
    if h.dtype != torch.bfloat16 or not h.is_contiguous() or h.shape[1] != mw.K or h.shape[0] != T * topk:
        raise ValueError("moe_down_bs: h must be contiguous bf16 [T*topk, K]")
    alloc = torch.zeros if zero else torch.empty
    out = alloc(topk, T, mw.N, dtype=torch.float32, device=h.device)
    _check(lib().la_bsmoe(mw.fmt, 2, mw.desc32().data_ptr(), mw.N, mw.K, mw.E, order.data_ptr(), off.data_ptr(), topk,
                          h.data_ptr(), h.shape[1], T, 1, wts.data_ptr(), out.data_ptr(), mw.N, T * mw.N, 0,
                          MOE_BS_VAR if var is None else var, _stream()), "la_bsmoe")
    return Partial(out)


MOE_GEMV = os.environ.get("LOCALAI_AMD_MOE_GEMV", "1") == "1"
MOE_GEMV_MAX_T = 2


def moe_gemv_ok(mw: MoEWeights, T: int) -> bool:
    """Decode of 1-2 tokens: the routed experts on the int8-dot GEMV path (gemv_dp4.hip
    moe_gemv_kernel) instead of the MFMA grouped GEMM, which pads each expert's 1-2 rows to 16."""
    return (MOE_GEMV and T <= MOE_GEMV_MAX_T and mw.desc is not None and mw.K % 256 == 0
            and mw.fmt in (FMT_Q4_K, FMT_Q6_K, FMT_Q8_0) and all(w.gemv_ok for w in mw.experts[:1]))


# split-K override of the MoE decode GEMVs (gate|up, down); 0: the dense GEMV's heuristic (A/B knob)
MOE_GEMV_SPLITS = tuple(int(v) for v in os.environ.get("LOCALAI_AMD_MOE_GEMV_SPLITS", "0,0").split(","))


def moe_gemv(x: Optional[torch.Tensor], mw: MoEWeights, ids: torch.Tensor, topk: int, T: int, E_local: int,
             act_src: Optional[Partial] = None, act_mode: int = ACT_SWIGLU,
             wts: Optional[torch.Tensor] = None) -> Partial:
    """gate|up (act_src None): x [T, K] -> Partial [S, T*topk, N] (row = routed pair); down
    (act_src = the gate|up Partial): x = wts[p] * act(gate|up row p) -> Partial [S*topk, T, N],
    the same slab contract as moe_linear.  ids: [T*topk] int32 local expert ids (>= E_local:
    another rank's expert, rows read as zero)."""
    P = T * topk
    S = _gemv_splits([mw.experts[0]], mw.K, 1)
    # one token: its topk routed pairs already multiply the down launch's grid -- half the dense
    # GEMV's splits (Mixtral C=1 8 -> 4: 295.4 -> 300.3 / 294.5 -> 298.5 tok/s; gate|up 2 -> 1
    # neutral; at C=2 quartering both measured 1.3 % slower; r5_mxs*_*.log)
    if T == 1 and act_src is not None:
        nsb = mw.K // 256
        S = max(1, S // 2)
        while nsb % S or (mw.K // S) * (1 + 4 / 16 + 4 / 32) > 65536:
            S += 1
    ov = MOE_GEMV_SPLITS[0 if act_src is None else 1]
    if ov > 0 and (mw.K // 256) % ov == 0 and (mw.K // ov) * (1 + 4 / 16 + 4 / 32) <= 65536:
        S = ov
    dev = ids.device
    if act_src is None:
        out = torch.empty(S, P, mw.N, dtype=torch.float32, device=dev)
        slab = P * mw.N
        _check(lib().la_moe_gemv(mw.fmt, 0, mw.desc.data_ptr(), mw.N, mw.K, E_local, ids.data_ptr(), T, topk,
                                 x.data_ptr(), x.shape[1], S, None, 0, 0, 0, None, out.data_ptr(), mw.N, slab,
                                 _stream()), "la_moe_gemv")
    else:
        a = act_src.src_args()
        if act_src.t.dim() != 3 or a[3]:
            raise ValueError("moe_gemv: the activation source must be fp32 slabs without bias")
        out = torch.empty(S * topk, T, mw.N, dtype=torch.float32, device=dev)
        slab = T * mw.N
        _check(lib().la_moe_gemv(mw.fmt, 1, mw.desc.data_ptr(), mw.N, mw.K, E_local, ids.data_ptr(), T, topk,
                                 None, 0, S, a[0], a[1], a[2], act_mode, wts.data_ptr(), out.data_ptr(), mw.N, slab,
                                 _stream()), "la_moe_gemv")
    return Partial(out)


def grammar_mask(logits: torch.Tensor, slot: torch.Tensor, pool: torch.Tensor) -> None:
    """In-place: logits[b, v] = -inf where pool[slot[b], v] == 0, for rows with slot[b] >= 0
    (grammar-constrained rows whose parse state has a cached allowed-token mask).  pool is
    [slots, >= V] uint8 / bool; slot [B] int32."""
    B, V = logits.shape
    assert pool.shape[1] >= V and slot.shape[0] >= B and slot.dtype == torch.int32
    if not logits.is_cuda:
        for b in range(B):
            s = int(slot[b])
            if s >= 0:
                logits[b].masked_fill_(~pool[s, :V].bool(), float("-inf"))
        return
    if logits.dtype != torch.float32 or logits.stride(1) != 1 or pool.stride(1) != 1:
        raise ValueError("grammar_mask: f32 logits and a row-major pool required")
    _check(lib().la_grammar_mask(logits.data_ptr(), logits.stride(0), B, V, slot.data_ptr(), pool.data_ptr(),
                                 pool.stride(0), _stream()), "la_grammar_mask")


def grammar_advance(tok: torch.Tensor, slot: torch.Tensor, nxt: torch.Tensor) -> None:
    """In-place: for rows with slot >= 0, slot = nxt[slot, tok] if that transition is known
    (>= 0) else -3 (parked: the host drops the row's later tokens of this run).  tok / slot
    int32 [B]; nxt int16 [slots, V]."""
    B = slot.shape[0]
    V = nxt.shape[1]
    assert nxt.dtype == torch.int16 and slot.dtype == torch.int32 and tok.shape[0] >= B
    if not slot.is_cuda:
        for b in range(B):
            s, t = int(slot[b]), int(tok[b])
            if s >= 0:
                ns = int(nxt[s, t]) if 0 <= t < V else -2
                slot[b] = ns if ns >= 0 else -3
        return
    _check(lib().la_grammar_advance(tok.data_ptr(), slot.data_ptr(), nxt.data_ptr(), V, B, _stream()),
           "la_grammar_advance")


def penalties(logits: torch.Tensor, hist: torch.Tensor, hist_len: torch.Tensor, pen: torch.Tensor,
              nl_token: int = -1, penalize_nl: Optional[torch.Tensor] = None, col0: int = 0):
    """In-place repeat/frequency/presence penalties.  hist [B, L] i32 (-1 padded); pen [B,3].
    col0 > 0 or a narrower row: logits hold the vocabulary columns [col0, col0 + V) only (a
    tensor-parallel shard); history tokens outside them are skipped."""
    B = logits.shape[0]
    if not logits.is_cuda:
        V = logits.shape[1]
        for b in range(B):
            L = int(hist_len[b])
            rp, fp, pp = (float(x) for x in pen[b])
            toks = hist[b, :L].tolist()
            for t in set(toks):
                if t < 0:
                    continue
                if t == nl_token and penalize_nl is not None and not bool(penalize_nl[b]):
                    continue
                if t < col0 or t - col0 >= V:
                    continue
                c = toks.count(t)
                v = float(logits[b, t - col0])
                if rp != 1:
                    v = v / rp if v > 0 else v * rp
                v -= c * fp + (pp if c > 0 else 0)
                logits[b, t - col0] = v
        return logits
    _check(lib().la_penalties_cols(logits.data_ptr(), logits.stride(0), B, hist.data_ptr(), hist.stride(0),
                                   hist_len.data_ptr(), pen.data_ptr(), nl_token, _ptr(penalize_nl), col0,
                                   logits.shape[1], _stream()), "la_penalties_cols")
    return logits


# Tensor-parallel sampling over vocabulary shards (sampling.hip tp_* kernels; decoder.TPInfo.sample_cols)
TP_SAMPLE_C = 64   # standard-chain candidates per rank and row: rows with 1 <= top_k <= TP_SAMPLE_C


def tp_topc(logits: torch.Tensor, C: int, base: int, out: torch.Tensor) -> None:
    """out [B, C, 2] f32 (this rank's slot of the exchange buffer): the C largest logits of each row
    of the shard as (value, global id), in increasing id order."""
    B, Vs = logits.shape
    _check(lib().la_tp_topc(logits.data_ptr(), logits.stride(0), B, Vs, C, base, out.data_ptr(), _stream()),
           "la_tp_topc")


def tp_mirostat(phase: int, logits: torch.Tensor, base: int, world: int, rank: int, params_dev: torch.Tensor,
                mu: torch.Tensor, x1: torch.Tensor, x2: torch.Tensor, x3: torch.Tensor, own: Optional[torch.Tensor],
                out_tok: Optional[torch.Tensor]) -> None:
    B, Vs = logits.shape
    _check(lib().la_tp_mirostat(phase, logits.data_ptr(), logits.stride(0), B, Vs, base, world, rank,
                                params_dev.data_ptr(), mu.data_ptr(), x1.data_ptr(), x2.data_ptr(), x3.data_ptr(),
                                _ptr(own), _ptr(out_tok), _stream()), "la_tp_mirostat")


def penalty_push(nxt: torch.Tensor, hist: torch.Tensor, cnt: torch.Tensor, hl: torch.Tensor,
                 cap: torch.Tensor) -> None:
    """Append the sampled tokens to each row's penalty ring (hist [B, L] i32, ring size cap[b])
    and refresh hist_len = min(count, cap) -- the in-graph history the penalties kernel reads."""
    B = nxt.shape[0]
    if not nxt.is_cuda:
        for b in range(B):
            k = int(cap[b])
            if k <= 0:
                continue
            c = int(cnt[b])
            hist[b, c % k] = nxt[b]
            cnt[b] = c + 1
            hl[b] = min(c + 1, k)
        return
    _check(lib().la_pen_push(nxt.data_ptr(), B, hist.data_ptr(), hist.stride(0), cnt.data_ptr(), hl.data_ptr(),
                             cap.data_ptr(), _stream()), "la_pen_push")


# ---------------------------------------------------------------------------------------
# Mamba decode step (mamba.hip)
# ---------------------------------------------------------------------------------------

def mamba_conv_step(conv_state: torch.Tensor, xz: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor],
                    out: torch.Tensor) -> torch.Tensor:
    """conv_state [B, I, K] fp32 (rolled in place); xz [B, >=2I] fp32; w [I, K] fp32 -> out [B, I]."""
    B, I, K = conv_state.shape
    for t in (conv_state, xz, w, out):
        assert t.dtype == torch.float32 and t.is_cuda and t.stride(-1) == 1
    assert conv_state.is_contiguous() and w.shape == (I, K) and out.shape == (B, I) and out.is_contiguous()
    assert xz.shape[0] == B and xz.shape[1] >= 2 * I and (bias is None or bias.shape == (I,))
    _check(lib().la_mamba_conv_step(conv_state.data_ptr(), xz.data_ptr(), xz.stride(0), w.data_ptr(),
                                    None if bias is None else bias.data_ptr(), out.data_ptr(), B, I, K, _stream()),
           "la_mamba_conv_step")
    return out


def mamba_ssm_step(ssm_state: torch.Tensor, x: torch.Tensor, dt: torch.Tensor, bc: torch.Tensor, off_b: int,
                   off_c: int, A: torch.Tensor, D: torch.Tensor, xz: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """Selective-state update of one token: ssm_state [B, I, N] fp32 (in place), x / dt [B, I],
    bc [B, *] holding B at off_b and C at off_c, A [I, N] (negative), D [I], z = xz[:, I:2I]."""
    B, I, N = ssm_state.shape
    for t in (ssm_state, x, dt, bc, A, D, xz, out):
        assert t.dtype == torch.float32 and t.is_cuda and t.stride(-1) == 1
    assert ssm_state.is_contiguous() and x.is_contiguous() and dt.is_contiguous() and out.is_contiguous()
    assert A.shape == (I, N) and D.shape == (I,) and bc.shape[0] == B and bc.shape[1] >= max(off_b, off_c) + N
    assert xz.shape[0] == B and xz.shape[1] >= 2 * I
    _check(lib().la_mamba_ssm_step(ssm_state.data_ptr(), x.data_ptr(), dt.data_ptr(), bc.data_ptr(), bc.stride(0),
                                   off_b, off_c, A.data_ptr(), D.data_ptr(), xz.data_ptr(), xz.stride(0),
                                   out.data_ptr(), B, I, N, _stream()), "la_mamba_ssm_step")
    return out


# ---------------------------------------------------------------------------------------
# GroupNorm (+ SiLU) over NHWC bf16 activations (groupnorm.hip) -- the SD UNet / VAE norms
# ---------------------------------------------------------------------------------------

def groupnorm_supported(x: torch.Tensor, groups: int) -> bool:
    if not (x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 4):
        return False
    C = x.shape[1]
    return (x.is_contiguous(memory_format=torch.channels_last) and groups <= 64 and 256 % (2 * groups) == 0
            and C % groups == 0
            and (C // groups) % 2 == 0 and C <= 2048)


# ---------------------------------------------------------------------------------------
# Image preprocessing (K26): PIL-exact bicubic resample + placement + normalise + tiles
# ---------------------------------------------------------------------------------------

def _bicubic(x: float) -> float:
    a = -0.5
    x = abs(x)
    if x < 1.0:
        return ((a + 2.0) * x - (a + 3.0)) * x * x + 1
    if x < 2.0:
        return (((x - 5) * x + 8) * x - 4) * a
    return 0.0


@functools.lru_cache(maxsize=64)
def pil_bicubic_coeffs(in_size: int, out_size: int) -> Tuple[np.ndarray, np.ndarray, int]:
    """PIL's precompute_coeffs + normalize_coeffs_8bpc for BICUBIC (Resample.c): per output
    index the first source index and count, and int32 weights in 22-bit fixed point."""
    scale = in_size / out_size
    filterscale = max(scale, 1.0)
    support = 2.0 * filterscale
    ksize = int(math.ceil(support)) * 2 + 1
    bounds = np.zeros((out_size, 2), dtype=np.int32)
    kk = np.zeros((out_size, ksize), dtype=np.int32)
    ss = 1.0 / filterscale
    for xx in range(out_size):
        center = (xx + 0.5) * scale
        xmin = max(int(center - support + 0.5), 0)
        xmax = min(int(center + support + 0.5), in_size) - xmin
        w = [_bicubic((x + xmin - center + 0.5) * ss) for x in range(xmax)]
        ww = sum(w)
        for x in range(xmax):
            c = w[x] / ww if ww != 0.0 else w[x]
            kk[xx, x] = int(-0.5 + c * (1 << 22)) if c < 0 else int(0.5 + c * (1 << 22))
        bounds[xx] = (xmin, xmax)
    return bounds, kk, ksize


_IMG_TABLES: dict = {}


def _img_tables(in_size: int, out_size: int, device):
    key = (in_size, out_size, str(device))
    t = _IMG_TABLES.get(key)
    if t is None:
        b, k, ks = pil_bicubic_coeffs(in_size, out_size)
        t = _IMG_TABLES[key] = (torch.from_numpy(b).to(device), torch.from_numpy(k).to(device), ks)
    return t


def image_tiles(img: torch.Tensor, placements: Sequence[dict], out: torch.Tensor, mean, std) -> torch.Tensor:
    """img: uint8 [H, W, 3] on the GPU.  Each placement resizes the image to (ow, oh) with PIL's
    BICUBIC (bit-exact), puts it at (ox, oy) on a (cw, ch) canvas filled with `fill`, and writes the
    canvas' S x S tiles, normalised, into out[t0 + i] (out: fp32 [n, 3, S, S])."""
    H, W, _ = img.shape
    S = out.shape[-1]
    assert img.dtype == torch.uint8 and img.is_contiguous() and out.is_contiguous() and out.dtype == torch.float32
    m = torch.tensor(list(mean), dtype=torch.float32, device=img.device)
    sd = torch.tensor(list(std), dtype=torch.float32, device=img.device)
    for pl in placements:
        ow, oh, cw, ch = int(pl["ow"]), int(pl["oh"]), int(pl["cw"]), int(pl["ch"])
        if cw % S or ch % S or pl["t0"] + (cw // S) * (ch // S) > out.shape[0]:
            raise ValueError("image_tiles: canvas does not tile the output")
        bh, kh, ksh = _img_tables(W, ow, img.device)
        bv, kv, ksv = _img_tables(H, oh, img.device)
        tmp = torch.empty(H, ow, 3, dtype=torch.uint8, device=img.device)
        _check(lib().la_img_resample_h(img.data_ptr(), H, W, tmp.data_ptr(), ow, bh.data_ptr(), kh.data_ptr(), ksh,
                                       _stream()), "la_img_resample_h")
        fill = torch.tensor(list(pl.get("fill", (0, 0, 0))), dtype=torch.int32, device=img.device)
        _check(lib().la_img_resample_v_tiles(tmp.data_ptr(), oh, ow, bv.data_ptr(), kv.data_ptr(), ksv, ch, cw,
                                             int(pl.get("oy", 0)), int(pl.get("ox", 0)), S, int(pl["t0"]),
                                             m.data_ptr(), sd.data_ptr(), fill.data_ptr(), out.data_ptr(), _stream()),
               "la_img_resample_v_tiles")
    return out


def groupnorm_nhwc(x: torch.Tensor, groups: int, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                   eps: float, silu: bool = False) -> torch.Tensor:
    """x [B, C, H, W] bf16 in channels_last memory -> GroupNorm(x) (SiLU'd when `silu`), same layout."""
    assert groupnorm_supported(x, groups), "groupnorm_nhwc: bf16 channels_last, even channels per group, C <= 2048"
    B, C, H, W = x.shape
    for t in (weight, bias):
        assert t is None or (t.dtype == torch.bfloat16 and t.is_contiguous() and t.numel() == C)
    HW = H * W
    rows_s = max(1, -(-HW * B // 256))    # statistics: ~256 workgroups, few partials
    rows_a = max(1, -(-HW * B // 1024))   # apply: ~1024 workgroups over the chip
    S = -(-HW // rows_s)
    part = torch.empty(B * S * groups * 2, dtype=torch.float32, device=x.device)
    y = torch.empty_like(x, memory_format=torch.channels_last)
    _check(lib().la_groupnorm_nhwc(x.data_ptr(), y.data_ptr(), _ptr(weight), _ptr(bias), part.data_ptr(), B, HW, C,
                                   groups, rows_s, rows_a, float(eps), int(silu), _stream()), "la_groupnorm_nhwc")
    return y
