"""Gosuvik: a decoder-only design described layer by layer in its config.json.

Pre-normed layers on an fp32 residual stream, x <- x + mixer(n1(x)), x <- x + ff(n2(x)) (ff
optional); the norm divides each of `norm.groups` equal parts of the vector by its own root mean
square and multiplies the whole by a weight (ops.add_group_norm: residual add and the next
sublayer's norm in one launch).  A span of layers may run several times in a row with the same
weights (`loop`); every pass is a layer RUN with K/V pages and state of its own.  Three mixers:

  * "channel_delta": the gated delta rule with one decay per head and key channel
    (ops.delta_rule): short convolutions with silu on q, k, v, unit-length q and k, a write
    strength beta, decays from a low-rank projection, S <- diag(g) S + k (beta (v - S^T k))^T,
    read-out after the write, unit norm per head and a low-rank sigmoid gate.  Convolution tail
    and the fp32 state are per-sequence state in the scheduler's slot pool;
  * "latent_attention": keys and values expanded from a normed latent row plus one rotated key
    part shared by the heads (ops.latent_kv, attn_mix over the latent pages with the per-head
    up-projections moved to the query and output sides), sliding window, YaRN-scaled rotation,
    an elementwise sigmoid gate on the concatenated heads (ops.sigmoid_mul);
  * "parallel": two mixers read the same input and their outputs are summed with fixed scales.
    Left: grouped-query attention with weighted per-head RMS norms on q and k, rotation with
    linearly scaled positions, values cached in the frame of their own position and the output
    turned back to the query's (ops.qk_norm_rope_pages, ops.rotate_heads), sliding window, a
    sink logit per head.  Right: a matrix memory with exponential gates under a running maximum
    (ops.matrix_memory), unit norm per head, sigmoid gate.  Both output projections are one GEMM
    over the concatenated, scaled branches.

Feed-forwards: down(poly(up h)) with a polynomial activation of unit powers (ops.poly_norm_act),
or routed experts down(silu(gate h) * up h) chosen by the largest softmax scores and weighted by
the chosen scores over their sum (ops.router_softmax: the same numbers).

The model plugs into LLMEngine like the other layer-list families: ForwardBatch, KVCache.layered,
the native scheduler's block tables and state slots; one query row per token, so prompt portions
and decoded tokens of different sequences share a forward (`mixed_batches`).  bf16 serving keeps
the residual stream, norms, angles, scores and softmax, routers, gates, decays, unit norms and the
recurrences with their state in fp32; dtype=torch.float32 serves in true fp32 end to end.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from .. import ops
from ..gguf import dequantize
from .decoder import ForwardBatch, KVCache, TPInfo

# routed experts: (token, expert) pair GEMVs up to this many rows, grouped rows + library GEMMs beyond
MOE_PAIR_MAX_T = int(os.environ.get("LOCALAI_AMD_GOSUVIK_PAIR_MAX_T", "32"))
# from this many rows on the grouped expert kernels give way to library GEMMs per expert
MOE_DENSE_MIN_T = 6144
DECODE_TILES = os.environ.get("LOCALAI_AMD_GOSUVIK_DECODE_TILES", "1") == "1"
DECODE_WGS = int(os.environ.get("LOCALAI_AMD_GOSUVIK_DECODE_WGS", "1024"))
UNIT_EPS = 1e-6      # inside the root of the delta rule's unit-length q and k
DENOM_EPS = 1e-6     # added to the matrix memory's denominator


@dataclass
class RotSpec:
    dims: int
    base: float
    scaling: Optional[dict] = None      # {"factor"}: positions divided by it; with "original", "fast", "slow": YaRN


@dataclass
class MixSpec:
    kind: str                 # "channel_delta" | "latent_attention" | "parallel" | "sink_attention" | "matrix_memory"
    heads: int = 0
    dim: int = 0              # query / key width per head (latent attention: the unrotated part)
    vdim: int = 0
    kv_heads: int = 0         # channel_delta: q / k heads; sink_attention: key / value heads
    taps: int = 0             # channel_delta: convolution taps
    rot: Optional[RotSpec] = None
    scale: float = 1.0
    window: int = 0           # keys i - window < j <= i (0: all)
    rot_dim: int = 0          # latent attention: rotated query / key width
    kv_rank: int = 0
    gate_cap: float = 0.0     # matrix_memory
    left: Optional["MixSpec"] = None
    right: Optional["MixSpec"] = None
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass
class FfSpec:
    kind: str                 # "dense" | "moe"
    ff: int
    experts: int = 0
    top: int = 0


@dataclass
class GosuvikHParams:
    n_vocab: int
    n_embd: int
    norm_eps: float
    norm_groups: int = 1
    mixers: List[MixSpec] = field(default_factory=list)
    mlps: List[Optional[FfSpec]] = field(default_factory=list)
    loop: Optional[Tuple[int, int, int]] = None     # (start, stop, times)
    arch: str = "gosuvik"
    name: str = ""

    @property
    def n_layer(self) -> int:
        return len(self.mixers)

    @property
    def runs(self) -> List[int]:
        """Layer indices in execution order (a looped span repeated)."""
        n = self.n_layer
        if not self.loop:
            return list(range(n))
        a, b, times = self.loop
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    @staticmethod
    def _rot(r: dict) -> RotSpec:
        return RotSpec(int(r["dims"]), float(r["base"]), dict(r["scaling"]) if r.get("scaling") else None)

    @staticmethod
    def _window(m: dict) -> int:
        return int((m.get("mask") or {}).get("size") or 0)

    @classmethod
    def _mixer(cls, kind: str, m: dict, where: str) -> MixSpec:
        if kind == "channel_delta":
            return MixSpec(kind, int(m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"]),
                           kv_heads=int(m.get("kv_heads") or m["heads"]), taps=int(m["conv"]))
        if kind == "latent_attention":
            return MixSpec(kind, int(m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"]), rot=cls._rot(m["rot"]),
                           scale=float(m["scale"]), window=cls._window(m), rot_dim=int(m["rot_dim"]),
                           kv_rank=int(m["kv_rank"]))
        if kind == "parallel":
            l, r = m["left"], m["right"]
            left = MixSpec("sink_attention", int(l["heads"]), int(l["dim"]), int(l.get("vdim") or l["dim"]),
                           kv_heads=int(l.get("kv_heads") or l["heads"]), rot=cls._rot(l["rot"]), scale=float(l["scale"]),
                           window=cls._window(l))
            right = MixSpec("matrix_memory", int(r["heads"]), int(r["dim"]), int(r.get("vdim") or r["dim"]),
                            gate_cap=float(r["gate_cap"]))
            return MixSpec(kind, left=left, right=right, left_scale=float(m["left_scale"]),
                           right_scale=float(m["right_scale"]))
        raise ValueError(f"{where}: unknown mixer type {kind!r}")

    @staticmethod
    def from_config(c: dict, name: str = "") -> "GosuvikHParams":
        hp = GosuvikHParams(n_vocab=int(c["vocab"]), n_embd=int(c["width"]), norm_eps=float(c["norm"]["eps"]),
                            norm_groups=int(c["norm"].get("groups") or 1), name=name)
        if hp.n_embd % hp.norm_groups:
            raise ValueError("norm.groups must divide the width")
        for i, L in enumerate(c["layers"]):
            hp.mixers.append(hp._mixer(L.get("type"), L["mixer"], f"layer {i}"))
            f = L.get("mlp")
            if not f:
                hp.mlps.append(None)
            elif f.get("kind") == "dense":
                hp.mlps.append(FfSpec("dense", int(f["ff"])))
            elif f.get("kind") == "moe":
                hp.mlps.append(FfSpec("moe", int(f["expert"]["ff"]), int(f["router"]["experts"]), int(f["router"]["top"])))
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
        lp = c.get("loop")
        if lp and int(lp.get("times", 1)) >= 1 and int(lp["stop"]) > int(lp["start"]):
            hp.loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
            if not 0 <= hp.loop[0] < hp.loop[1] <= hp.n_layer:
                raise ValueError("loop: start / stop outside the layer list")
        return hp


@dataclass
class _Expert:
    gate_up: ops.QWeight
    down: ops.QWeight


@dataclass
class _Layer:
    norm1: torch.Tensor
    win: ops.QWeight                   # the mixer's fused input projections (see the loaders)
    wo: ops.QWeight
    norm2: Optional[torch.Tensor] = None
    # channel_delta
    a2: Optional[ops.QWeight] = None
    g2: Optional[ops.QWeight] = None
    rank_a: int = 0
    rank_g: int = 0
    conv: Optional[torch.Tensor] = None          # fp32 [C, taps]
    conv_t: Optional[torch.Tensor] = None        # the same tap-major, [taps, C] (the vectorised kernel's layout)
    dt_bias: Optional[torch.Tensor] = None
    a_log: Optional[torch.Tensor] = None
    mix_norm: Optional[torch.Tensor] = None
    # attention mixers
    freqs: Optional[torch.Tensor] = None
    mag: float = 1.0
    dkv_norm: Optional[torch.Tensor] = None
    uk: Optional[torch.Tensor] = None            # [H, dim, kv_rank] activation dtype
    uv_t: Optional[torch.Tensor] = None          # [H, kv_rank, vdim]
    q_norm: Optional[torch.Tensor] = None
    k_norm: Optional[torch.Tensor] = None
    v_freqs: Optional[torch.Tensor] = None
    sink: Optional[torch.Tensor] = None
    # matrix memory
    gate_b: Optional[torch.Tensor] = None        # fp32 [2 H]: input | forget biases
    mem_norm: Optional[torch.Tensor] = None
    # feed-forward
    up: Optional[ops.QWeight] = None
    down: Optional[ops.QWeight] = None
    poly: Optional[torch.Tensor] = None          # fp32 [4]
    router: Optional[torch.Tensor] = None        # fp32 [E, D]
    wg: Optional[torch.Tensor] = None            # stacked expert weights [E, F, D] / [E, D, F], activation dtype
    wu: Optional[torch.Tensor] = None
    wd: Optional[torch.Tensor] = None
    experts: Optional[List[_Expert]] = None
    moe_gu: Optional[object] = None              # ops.MoEWeights where the grouped expert GEMMs take the shape
    moe_down: Optional[object] = None


class GosuvikModel:
    # what this family launches from ops/csrc (ops.require_kernels: a first run compiles only these)
    kernel_sources = ("elementwise.hip", "norm_chain.hip", "rope_pages.hip", "retention.hip", "delta_rule.hip",
                      "matrix_memory.hip", "attention_mix.hip", "attention.hip", "attention_latent.hip", "moe_dense.hip",
                      "moe.hip", "sampling.hip", "decode_loop.hip", "gemm_skinny.hip")
    stateful = True         # convolution tails and recurrent state per sequence: state slots, no prefix-cache reuse
    mixed_batches = True    # prompt portions and decode rows of different sequences in one forward

    def __init__(self, reader, device: torch.device, tp: Optional[TPInfo] = None, max_pos: Optional[int] = None,
                 rope_overrides: Optional[dict] = None, lora=None, dtype: torch.dtype = torch.bfloat16):
        self.tp = tp or TPInfo()
        if self.tp.world > 1:
            raise ValueError("gosuvik: tensor parallelism is not implemented for this design")
        if lora is not None:
            raise ValueError("gosuvik: LoRA adapters are not supported")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("gosuvik: serving dtype is bfloat16 or float32")
        self.device, self.dtype = device, dtype
        self.f32 = dtype == torch.float32
        self.hp = hp = GosuvikHParams.from_config(reader.config, str(reader.kv.get("general.name", "")))
        self.max_pos = max_pos or 1 << 20
        self.vocab_local = hp.n_vocab
        self.T = reader.tensors
        D = hp.n_embd
        self.tok_embd = ops.QWeight.from_float(self._shaped("embed", (hp.n_vocab, D)).to(device))   # bf16 table, exact
        self.layers: List[_Layer] = []
        loaders = {"channel_delta": self._load_delta, "latent_attention": self._load_latent, "parallel": self._load_parallel}
        for i, (m, f) in enumerate(zip(hp.mixers, hp.mlps)):
            p = f"l{i}."
            L = loaders[m.kind](p + "mix.", m)
            L.norm1 = self._f32(p + "norm1", (D,))
            if f is not None:
                L.norm2 = self._f32(p + "norm2", (D,))
                self._load_ff(L, p + "mlp.", f)
            self.layers.append(L)
        self.out_norm = self._f32("final.norm", (D,))
        self.output = self._qw(self._shaped("head", (hp.n_vocab, D)))
        self._aranges: Dict[int, tuple] = {}
        self.T = None

    # --------------------------------------------------------------------------- loading
    def _raw(self, name: str) -> torch.Tensor:
        if name not in self.T:
            raise KeyError(f"gosuvik: missing tensor {name}")
        t = self.T[name]
        return torch.from_numpy(dequantize(t.data, t.ggml_type, t.shape).astype(np.float32).reshape(t.shape))

    def _shaped(self, name: str, shape) -> torch.Tensor:
        w = self._raw(name)
        if tuple(w.shape) != tuple(shape):
            raise ValueError(f"gosuvik: {name} is {tuple(w.shape)}, the config asks for {tuple(shape)}")
        return w

    def _f32(self, name: str, shape) -> torch.Tensor:
        return self._shaped(name, shape).to(self.device).contiguous()

    def _qw(self, w: torch.Tensor) -> ops.QWeight:
        w = w.to(self.device)
        return ops.QWeight.from_f32(w) if self.f32 else ops.QWeight.from_float(w)

    def _freqs(self, r: RotSpec):
        """(frequencies, magnitude) of a rotation: YaRN when the scaling names an original length,
        positions divided by the factor when it gives a factor alone."""
        s = r.scaling
        if s and "original" in s:
            return ops.rot_freqs(r.dims, r.base, s, self.device)
        return ops.linear_rot_freqs(r.dims, r.base, float(s["factor"]) if s else 1.0, self.device), 1.0

    def _load_delta(self, p: str, m: MixSpec) -> _Layer:
        D, H, G = self.hp.n_embd, m.heads, m.kv_heads
        sh = self._shaped
        if H % G or m.taps < 1:
            raise ValueError(f"{p}: heads must be a multiple of kv_heads, conv at least 1")
        Cqk, Cv = G * m.dim, H * m.vdim
        a1, g1 = self._raw(p + "a1"), self._raw(p + "g1")
        if a1.dim() != 2 or g1.dim() != 2 or a1.shape[1] != D or g1.shape[1] != D:
            raise ValueError(f"{p}: a1 / g1 read the layer's input")
        ra, rg = a1.shape[0], g1.shape[0]
        win = torch.cat([sh(p + "q", (Cqk, D)), sh(p + "k", (Cqk, D)), sh(p + "v", (Cv, D)), sh(p + "b", (H, D)), a1, g1], 0)
        if win.shape[0] % 8:     # rows of zeros up to a multiple of 8: the projection's rows stay 16-byte aligned in bf16
            win = torch.cat([win, torch.zeros(8 - win.shape[0] % 8, D)], 0)
        L = _Layer(None, self._qw(win), self._qw(sh(p + "o", (D, Cv))))
        L.a2, L.g2 = self._qw(sh(p + "a2", (H * m.dim, ra))), self._qw(sh(p + "g2", (Cv, rg)))
        L.rank_a, L.rank_g = ra, rg
        L.conv = torch.cat([sh(p + "q.conv", (Cqk, m.taps)), sh(p + "k.conv", (Cqk, m.taps)),
                            sh(p + "v.conv", (Cv, m.taps))], 0).to(self.device).contiguous()
        L.conv_t = L.conv.t().contiguous()
        L.dt_bias = self._f32(p + "dt_bias", (H * m.dim,))
        L.a_log = self._f32(p + "A_log", (H,))
        L.mix_norm = self._f32(p + "norm", (m.vdim,))
        return L

    def _load_latent(self, p: str, m: MixSpec) -> _Layer:
        D, H = self.hp.n_embd, m.heads
        sh = self._shaped
        if m.rot.dims != m.rot_dim or m.rot_dim % 2:
            raise ValueError(f"{p}: rot.dims must equal rot_dim (even)")
        win = torch.cat([sh(p + "q", (H * (m.dim + m.rot_dim), D)), sh(p + "dkv", (m.kv_rank + m.rot_dim, D)),
                         sh(p + "g", (H * m.vdim, D))], 0)
        L = _Layer(None, self._qw(win), self._qw(sh(p + "o", (D, H * m.vdim))))
        L.freqs, L.mag = self._freqs(m.rot)
        L.dkv_norm = self._f32(p + "dkv.norm", (m.kv_rank,))
        L.uk = sh(p + "uk", (H * m.dim, m.kv_rank)).view(H, m.dim, m.kv_rank).to(self.device, self.dtype).contiguous()
        L.uv_t = (sh(p + "uv", (H * m.vdim, m.kv_rank)).view(H, m.vdim, m.kv_rank).transpose(1, 2)
                  .to(self.device, self.dtype).contiguous())
        return L

    def _load_parallel(self, p: str, m: MixSpec) -> _Layer:
        D = self.hp.n_embd
        sh = self._shaped
        l, r = m.left, m.right
        if l.heads % l.kv_heads or l.rot.dims > l.dim or l.rot.dims % 2 or l.vdim % 2:
            raise ValueError(f"{p}left: heads a multiple of kv_heads, rot.dims even and at most dim, vdim even")
        pl, pr = p + "left.", p + "right."
        Hr = r.heads
        win = torch.cat([sh(pl + "q", (l.heads * l.dim, D)), sh(pl + "k", (l.kv_heads * l.dim, D)),
                         sh(pl + "v", (l.kv_heads * l.vdim, D)),
                         sh(pr + "q", (Hr * r.dim, D)), sh(pr + "k", (Hr * r.dim, D)), sh(pr + "v", (Hr * r.vdim, D)),
                         sh(pr + "g", (Hr * r.vdim, D)), sh(pr + "i", (Hr, D)), sh(pr + "f", (Hr, D))], 0)
        # both output projections as one GEMM over [left heads | right heads] (the branch scales
        # are applied to the activations, the stored weights stay exact)
        wo = torch.cat([sh(pl + "o", (D, l.heads * l.vdim)), sh(pr + "o", (D, Hr * r.vdim))], 1)
        L = _Layer(None, self._qw(win), self._qw(wo))
        L.freqs, L.mag = self._freqs(l.rot)
        L.v_freqs = ops.linear_rot_freqs(l.vdim, l.rot.base, 1.0, self.device)
        L.q_norm, L.k_norm = self._f32(pl + "q.norm", (l.dim,)), self._f32(pl + "k.norm", (l.dim,))
        L.sink = self._f32(pl + "sink", (l.heads,))
        L.gate_b = torch.cat([sh(pr + "i.b", (Hr,)), sh(pr + "f.b", (Hr,))]).to(self.device).contiguous()
        L.mem_norm = self._f32(pr + "norm", (Hr * r.vdim,))
        return L

    def _load_ff(self, L: _Layer, p: str, f: FfSpec) -> None:
        D, qw, sh = self.hp.n_embd, self._qw, self._shaped
        if f.kind == "dense":
            L.up, L.down = qw(sh(p + "up", (f.ff, D))), qw(sh(p + "down", (D, f.ff)))
            L.poly = self._f32(p + "act", (4,))
            return
        if not 1 <= f.top <= f.experts:
            raise ValueError(f"{p}: top must lie in 1 .. experts")
        L.router = self._f32(p + "router", (f.experts, D))
        ws = [(sh(p + f"e{e}.gate", (f.ff, D)), sh(p + f"e{e}.up", (f.ff, D)), sh(p + f"e{e}.down", (D, f.ff)))
              for e in range(f.experts)]
        L.wg, L.wu, L.wd = (torch.stack([w[k] for w in ws]).to(device=self.device, dtype=self.dtype).contiguous()
                            for k in range(3))
        L.experts = [_Expert(qw(torch.cat([g, u], 0)), qw(d)) for g, u, d in ws]
        if not self.f32 and self.device.type == "cuda" and D % 256 == 0 and f.ff % 256 == 0:
            # the framework's grouped expert GEMMs (one weight stream per active expert, device
            # routing, no host sync) read [gate; up] fused per expert
            L.moe_gu = ops.MoEWeights([e.gate_up for e in L.experts])
            L.moe_down = ops.MoEWeights([e.down for e in L.experts])

    # --------------------------------------------------------------------------- engine interface
    def _run_specs(self):
        """KVCache.layered spec of every layer run: (convolution tail, recurrent state) for a delta
        layer, latent pages for latent attention, K / V pages plus (memory, maximum) for a parallel layer."""
        out = []
        for i in self.hp.runs:
            m = self.hp.mixers[i]
            if m.kind == "channel_delta":
                C = 2 * m.kv_heads * m.dim + m.heads * m.vdim
                out.append((0, 0, 0, [((max(m.taps - 1, 0), C), None), ((m.heads, m.vdim, m.dim), torch.float32)]))
            elif m.kind == "latent_attention":
                out.append((1, m.kv_rank + m.rot_dim, 0, None))
            else:
                l, r = m.left, m.right
                out.append((l.kv_heads, l.dim, l.vdim, [((r.heads, r.vdim + 1, r.dim), torch.float32),
                                                        ((r.heads,), torch.float32)]))
        return out

    def kv_bytes_per_token(self) -> int:
        es = 4 if self.f32 else 2
        return max(es, sum(g * (dk + dv) * es for g, dk, dv, *_ in self._run_specs()))

    def new_kv_cache(self, num_blocks: int, block_size: int, state_slots: int = 0) -> KVCache:
        return KVCache.layered(self._run_specs(), num_blocks, block_size, self.device, self.dtype, state_slots)

    def decode_workspace(self, Bp: int, ctx: int, block_size: int):
        """Split-KV buffers of the decode attention kernel per (heads, kv heads, width) of the layers it serves."""
        out = {}
        for m in self.hp.mixers:
            l = m.left
            if l is not None and self._decode_kernel_ok(l, block_size):
                key = (l.heads, l.kv_heads, l.dim)
                if key not in out:
                    out[key] = ops.decode_workspace(Bp, l.heads, l.kv_heads, l.dim, ctx, self.device, block_size)
        return out or None

    def _decode_kernel_ok(self, l: MixSpec, block_size: int) -> bool:
        """Decode batches of this attention on the framework's split-KV decode attention kernel (the llama
        families'): bf16, equal key and value widths it is instantiated for; it takes the window and the sink."""
        return (not self.f32 and self.device.type == "cuda" and l.dim == l.vdim and l.dim in (64, 80, 96, 128, 192, 256)
                and l.heads // l.kv_heads <= 16 and block_size % 16 == 0 and (128 % block_size == 0 or block_size % 128 == 0)
                and ops._has("la_attn_decode"))

    def _prefill_kernel_ok(self, l: MixSpec) -> bool:
        """Batches of prompt portions only, for this attention, on the framework's prefill attention kernel
        (64 query rows of one head per workgroup): bf16, equal key and value widths it is instantiated for."""
        return (not self.f32 and self.device.type == "cuda" and l.dim == l.vdim and l.dim in (64, 80, 96, 128, 192, 256)
                and ops._has("la_attn_prefill"))

    def prefill_tiles(self, q_lens, device):
        """((16-row work tiles of the leading prompt portions for ops.attn_mix, 64-row tiles of the same
        portions for ops.attn_prefill where a layer has the widths that kernel takes), rows they cover)."""
        if device.type != "cuda" or self.f32:
            return None, 0
        mix, rows = ops.attn_mix_tiles(q_lens, device)
        pf = None
        if any(m.left is not None and self._prefill_kernel_ok(m.left) for m in self.hp.mixers):
            pf = ops.prefill_tiles(q_lens, device)
        return (mix, pf), rows

    def _single_rows(self, T: int):
        """(row -> sequence, row ranges, one-row work tiles) of a batch with one row per sequence."""
        a = self._aranges.get(T)
        if a is None:
            r = torch.arange(T + 1, dtype=torch.int32, device=self.device)
            tiles = torch.stack([r[:T], torch.zeros_like(r[:T])], 1).contiguous()
            a = self._aranges[T] = (r[:T].contiguous(), r, tiles)
        return a

    # --------------------------------------------------------------------------- forward
    def _dense(self, p: ops.Partial) -> torch.Tensor:
        """A projection's rows as one contiguous [T, N] matrix of the activation dtype."""
        t = p.t
        if p.bias is None and t.dim() == 3 and t.shape[0] == 1:
            t = t[0]
        elif p.bias is not None or t.dim() == 3:
            if t.is_cuda and p.N % 4 == 0:
                return ops.reduce(p, dtype=self.dtype)
            t = p.dense()
        return t if t.dtype == self.dtype else t.to(self.dtype)

    def _delta(self, L: _Layer, m: MixSpec, xn, fb, kv, run, cu_q):
        proj = self._dense(ops.linear(xn, L.win))            # [T, q | k | v | beta | decay rank | gate rank]
        c0 = 2 * m.kv_heads * m.dim + m.heads * m.vdim + m.heads
        dec = self._dense(ops.linear(proj[:, c0:c0 + L.rank_a].contiguous(), L.a2))
        gate = self._dense(ops.linear(proj[:, c0 + L.rank_a:c0 + L.rank_a + L.rank_g].contiguous(), L.g2))
        conv_state, rec_state = kv.state[run]
        return ops.delta_rule(proj, dec, gate, m.heads, m.kv_heads, m.dim, m.vdim, L.conv, L.dt_bias, L.a_log, L.mix_norm,
                              self.hp.norm_eps, fb.pos, cu_q, fb.sslots, conv_state, rec_state, UNIT_EPS,
                              max_rows=1 if fb.decode else fb.max_q, conv_wt=L.conv_t)

    def _latent(self, L: _Layer, m: MixSpec, xn, fb, kv, run, row_seq, splits: int = 1):
        T, H, r, dn, dr = xn.shape[0], m.heads, m.kv_rank, m.dim, m.rot_dim
        Cq = H * (dn + dr)
        proj = self._dense(ops.linear(xn, L.win))                     # [T, q | kv latent + rotated key | gate]
        q = ops.rope_pages(proj[:, :Cq].contiguous(), H, dn + dr, 0, 0, 0, fb.pos, None, L.freqs, L.mag, dr, dn,
                           False).view(T, H, dn + dr)
        ops.latent_kv(proj[:, Cq:Cq + r + dr].contiguous(), r, L.dkv_norm, self.hp.norm_eps, fb.pos, fb.slots, L.freqs,
                      L.mag, kv.k[run], interleaved=False)
        # the key up-projection moves to the query side: (W_uk c) . q = c . (W_uk^T q)
        qf = torch.empty(T, H, r + dr, dtype=self.dtype, device=xn.device)
        qf[:, :, :r] = torch.bmm(q[:, :, :dn].transpose(0, 1), L.uk).transpose(0, 1)
        qf[:, :, r:] = q[:, :, dn:]
        a = ops.attn_mix(qf.view(T, H * (r + dr)), kv.k[run], None, row_seq, fb.pos, fb.block_tables, H, m.scale,
                         window=m.window, v_width=r, key_splits=splits)
        # ... and the value up-projection to the output side: sum_j p_j W_uv c_j = W_uv sum_j p_j c_j
        o = torch.bmm(a.view(T, H, r).transpose(0, 1), L.uv_t).transpose(0, 1).reshape(T, H * m.vdim)
        return ops.sigmoid_mul(o, proj[:, Cq + r + dr:Cq + r + dr + H * m.vdim])

    def _sink_attention(self, L: _Layer, l: MixSpec, src, fb, kv, run, row_seq, cu_q, tiles, tile_rows, splits, ws):
        q = ops.qk_norm_rope_pages(src, l.heads, l.dim, l.kv_heads, l.vdim, fb.pos, fb.slots, L.q_norm, L.k_norm,
                                   self.hp.norm_eps, L.freqs, L.mag, l.rot.dims, L.v_freqs, kv.k[run], kv.v[run])
        T = q.shape[0]
        if fb.decode and fb.seq_lens is not None and self._decode_kernel_ok(l, kv.block_size):
            return ops.attn_decode(q.view(T, l.heads, l.dim), kv.k[run], kv.v[run], fb.block_tables, fb.seq_lens, l.scale,
                                   fb.max_len, workspace=ws, window=l.window, sink=L.sink).view(T, l.heads * l.vdim)
        if isinstance(tiles, tuple):
            tiles, pf = tiles
            if (pf is not None and not fb.decode and tile_rows == T and fb.ctx_lens is not None
                    and self._prefill_kernel_ok(l) and kv.block_size % 16 == 0):
                return ops.attn_prefill(q.view(T, l.heads, l.dim), kv.k[run], kv.v[run], cu_q, fb.ctx_lens, fb.block_tables,
                                        l.scale, window=l.window, tiles=pf, sink=L.sink).view(T, l.heads * l.vdim)
        return ops.attn_mix(q, kv.k[run], kv.v[run], row_seq, fb.pos, fb.block_tables, l.heads, l.scale, window=l.window,
                            tiles=tiles, tile_rows=tile_rows, cu_q=cu_q, key_splits=splits, sink=L.sink)

    def _parallel(self, L: _Layer, m: MixSpec, xn, fb, kv, run, row_seq, cu_q, tiles, tile_rows, splits, ws):
        l, r = m.left, m.right
        T = xn.shape[0]
        proj = self._dense(ops.linear(xn, L.win))            # [T, left q | k | v | right q | k | v | gate | i | f]
        wl = (l.heads + l.kv_heads) * l.dim + l.kv_heads * l.vdim
        nl = l.heads * l.vdim
        both = torch.empty(T, nl + r.heads * r.vdim, dtype=self.dtype, device=xn.device)
        a = self._sink_attention(L, l, proj, fb, kv, run, row_seq, cu_q, tiles, tile_rows, splits, ws)
        ops.rotate_heads(a, l.heads, l.vdim, fb.pos, L.v_freqs, -1.0, m.left_scale, out=both, col0=0)
        mem, mx = kv.state[run]
        ops.matrix_memory(proj[:, wl:], r.heads, r.dim, r.vdim, L.gate_b, r.gate_cap, L.mem_norm, self.hp.norm_eps, fb.pos,
                          cu_q, fb.sslots, mem, mx, scale=m.right_scale, denom_eps=DENOM_EPS,
                          max_rows=1 if fb.decode else fb.max_q, out=both, col0=nl)
        return both

    def _unit(self, x: torch.Tensor, e: _Expert, ff: int):
        """One gated expert on rows x: down(silu(gate x) * up x)."""
        gu = ops.linear(x, e.gate_up)
        if not self.f32 and (ff % 4 == 0 or not x.is_cuda):
            h = ops.act(gu, ff, ops.ACT_SWIGLU)
        else:
            g = self._dense(gu).float()
            h = (torch.nn.functional.silu(g[:, :ff]) * g[:, ff:]).to(self.dtype)
        return ops.linear(h, e.down)

    def _routed(self, L: _Layer, f: FfSpec, xn: torch.Tensor):
        """The weighted sum of every row's chosen experts (fp32 [T, D], or a Partial of it)."""
        T = xn.shape[0]
        ids, wts = ops.router_softmax(xn, L.router, None, f.top)
        capturing = xn.is_cuda and torch.cuda.is_current_stream_capturing()
        if L.moe_gu is not None and (T < MOE_DENSE_MIN_T or capturing) and T > 2:
            order, off = ops.moe_route(ids, f.experts)
            gu = ops.moe_linear(xn, L.moe_gu, order, off, f.top, T)
            h = ops.act(gu, f.ff, ops.ACT_SWIGLU)
            return ops.moe_linear(h, L.moe_down, order, off, f.top, T, down=True, wts=wts)
        if T <= MOE_PAIR_MAX_T or capturing:
            return ops.moe_pairs(xn, L.wg, L.wu, L.wd, ids, wts)
        # rows grouped by expert (device), one host read of the group offsets, then per expert
        # gate|up and down as library GEMMs over its rows and a weighted scatter-add in fp32
        order, off = ops.moe_route(ids, f.experts)
        off_h = off.cpu().tolist()
        order_l = order.long()
        tok = order_l // f.top
        xs = xn.index_select(0, tok)
        wsel = wts.index_select(0, order_l)
        out = torch.zeros(T, self.hp.n_embd, dtype=torch.float32, device=xn.device)
        with ops.blas_tuning_paused():
            for e in range(f.experts):
                r0, r1 = off_h[e], off_h[e + 1]
                if r1 <= r0:
                    continue
                y = self._dense(self._unit(xs[r0:r1].contiguous(), L.experts[e], f.ff)).float()
                out.index_add_(0, tok[r0:r1], y * wsel[r0:r1].unsqueeze(1))
        return out

    def _mlp(self, L: _Layer, f: FfSpec, xn: torch.Tensor):
        if f.kind == "dense":
            return ops.linear(ops.poly_norm_act(ops.linear(xn, L.up), L.poly, self.hp.norm_eps, self.dtype), L.down)
        return self._routed(L, f, xn)

    def forward(self, fb: ForwardBatch, kv: KVCache, attn_workspace=None, return_hidden: bool = False,
                local_logits: bool = False, layer_out: Optional[list] = None) -> torch.Tensor:
        """fp32 logits [R, V] of the rows fb.logits_idx selects (all rows when None).  Rows of one
        sequence are consecutive; fb.decode batches bring one row per sequence (fb.sslots per row),
        other batches fb.cu_q / fb.row_seq / fb.sslots per sequence.  layer_out: a list that
        receives the fp32 residual stream after every layer run (diagnostics)."""
        hp = self.hp
        T = fb.tokens.shape[0]
        if fb.sslots is None or kv.state is None:
            raise ValueError("gosuvik: the batch needs state slots (engine built without a state pool?)")
        if fb.decode:
            row_seq, cu_q, tiles = self._single_rows(T)
            tile_rows = T if (DECODE_TILES and not self.f32 and fb.tokens.is_cuda) else 0
            splits_for = lambda w: max(1, min(32, DECODE_WGS // max(T, 1), -(-(w or fb.max_len or 1) // 32)))  # noqa: E731
        else:
            row_seq, cu_q, tiles, tile_rows = fb.row_seq, fb.cu_q, fb.tiles, fb.tile_rows
            if row_seq is None:
                raise ValueError("gosuvik: prompt batches need fb.row_seq")
            splits_for = lambda w: 1  # noqa: E731
        if fb.tokens.is_cuda and hp.n_embd % 8:   # the embedding kernel reads 8 columns per thread
            res = self.tok_embd.materialize_bf16().index_select(0, fb.tokens.long()).float()
        else:
            res = ops.embed(fb.tokens, self.tok_embd)
        if not res.is_contiguous() or res.dtype != torch.float32:
            res = res.float().contiguous()
        runs = hp.runs
        eps, groups = hp.norm_eps, hp.norm_groups
        nc = lambda branch, w: ops.add_group_norm(res, branch, w, eps, groups, out_dtype=self.dtype)  # noqa: E731
        xn = nc(None, self.layers[runs[0]].norm1 if runs else self.out_norm)
        for r, i in enumerate(runs):
            L, m, f = self.layers[i], hp.mixers[i], hp.mlps[i]
            if m.kind == "channel_delta":
                a = self._delta(L, m, xn, fb, kv, r, cu_q)
            elif m.kind == "latent_attention":
                a = self._latent(L, m, xn, fb, kv, r, row_seq, splits_for(m.window))
            else:
                l = m.left
                ws = attn_workspace.get((l.heads, l.kv_heads, l.dim)) if isinstance(attn_workspace, dict) else None
                a = self._parallel(L, m, xn, fb, kv, r, row_seq, cu_q, tiles, tile_rows, splits_for(l.window), ws)
            o = ops.linear(a, L.wo)
            after = self.layers[runs[r + 1]].norm1 if r + 1 < len(runs) else self.out_norm
            if f is not None:
                xn = nc(o, L.norm2)
                xn = nc(self._mlp(L, f, xn), after)
            else:
                xn = nc(o, after)
            if layer_out is not None:
                layer_out.append(res.clone())
        if return_hidden:
            return xn
        rows = xn if fb.logits_idx is None else xn.index_select(0, fb.logits_idx)
        lp = ops.linear(rows.contiguous(), self.output)
        return lp.t[0] if (lp.t.dim() == 3 and lp.t.shape[0] == 1 and lp.t.dtype == torch.float32) else self._dense(lp).float()
