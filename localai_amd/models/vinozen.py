"""Vinozen: a decoder-only design described layer by layer in its config.json.

The residual stream is normed on the sublayer's OUTPUT only: x <- x + ln1(mixer(x)), x <- x +
ln2(ff(x)) (ff optional), ln a layer norm with a weight and no bias; the sublayers read x itself
(ops.norm_chain with the "ln" norm after the branch and a plain cast before the next one).  A layer
ends with the per-layer token input shared with the other layer-list families (ops.side_gate: a
slice of a second embedding table gated by gelu(Wg x), projected, unit-normed, added).  The
embedding is scaled and gets additive sinusoidal positions (ops.sinusoid_add); the output is the
model's norm and the embedding table itself as the head.  Two mixers:

  * "attention": grouped-query softmax attention without rotation.  Queries and keys are divided by
    their root mean square per head, queries also multiplied by a temperature that grows with the
    logarithm of the position (ops.qk_norm_pages, which also appends K / V to the pages); scores
    get a learned bias per bucketed distance (ops.bucketed_bias -> attn_mix dist_bias) and the
    softmax a learned sink logit per head (attn_mix sink).  A layer with `kv_from` has no key /
    value projections and attends over the pages of the layer it names;
  * "mamba2": a state-space mixer with one decay per head (ops.mamba2): short convolution on
    [x | B | C], softplus step sizes, the N x P recurrence per head, silu(z) gate, grouped unit
    norm.  Convolution tail and recurrent state (fp32) are per-sequence state in the scheduler's
    slot pool.

Feed-forwards: SwiGLU, or routed experts of the clamped gated unit (ops.glu_clamp) chosen by the
largest router logits and weighted by the softmax over the chosen logits (ops.router_softmax), plus
a shared expert that runs for every token.

The model plugs into LLMEngine like the other layer-list families: ForwardBatch, KVCache.layered,
the native scheduler's block tables and state slots; one query row per token, so prompt portions
and decoded tokens of different sequences share a forward (`mixed_batches`).  bf16 serving keeps
the residual stream, norms, positions, scores and softmax, routers, step sizes, decays and the
recurrence in fp32; dtype=torch.float32 serves in true fp32 end to end.
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
MOE_PAIR_MAX_T = int(os.environ.get("LOCALAI_AMD_VINOZEN_PAIR_MAX_T", "32"))
# from this many rows on the grouped expert kernels give way to library GEMMs per expert
MOE_DENSE_MIN_T = 6144
DECODE_TILES = os.environ.get("LOCALAI_AMD_VINOZEN_DECODE_TILES", "1") == "1"
DECODE_WGS = int(os.environ.get("LOCALAI_AMD_VINOZEN_DECODE_WGS", "1024"))


@dataclass
class MixSpec:
    kind: str                 # "attention" | "mamba2"
    heads: int
    vdim: int                 # value width per head (mamba2: the head's channel count P)
    dim: int = 0              # attention: query / key width per head
    kv_heads: int = 0
    scale: float = 1.0
    temp_coef: float = 0.0    # query temperature 1 + coef ln(floor((p + 1) / every) + 1); every 0: none
    temp_every: int = 0
    bias_max: int = 0         # distances from here on share the last bias bucket
    kv_from: int = -1         # attention over this layer's pages (-1: its own)
    state: int = 0            # mamba2: N
    groups: int = 0           # mamba2: B / C groups
    taps: int = 0             # mamba2: convolution taps
    norm_groups: int = 1


@dataclass
class FfSpec:
    kind: str                 # "dense" | "moe"
    ff: int                   # dense: hidden width; moe: an expert's hidden width
    limit: float = 0.0        # experts: clamp of the gated unit
    experts: int = 0
    top: int = 0
    shared_ff: int = 0        # 0: no shared expert
    shared_limit: float = 0.0


@dataclass
class VinozenHParams:
    n_vocab: int
    n_embd: int
    norm_eps: float
    embed_scale: float = 1.0
    mixers: List[MixSpec] = field(default_factory=list)
    mlps: List[Optional[FfSpec]] = field(default_factory=list)
    side_dim: int = 0
    arch: str = "vinozen"
    name: str = ""

    @property
    def n_layer(self) -> int:
        return len(self.mixers)

    @staticmethod
    def from_config(c: dict, name: str = "") -> "VinozenHParams":
        hp = VinozenHParams(n_vocab=int(c["vocab"]), n_embd=int(c["width"]), norm_eps=float(c["norm"]["eps"]),
                            embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                            side_dim=int((c.get("token_side") or {}).get("dim") or 0), name=name)
        for i, L in enumerate(c["layers"]):
            m, kind = L["mixer"], L.get("type")
            if kind == "attention":
                qt = m.get("q_temp") or {}
                src = m.get("kv_from")
                hp.mixers.append(MixSpec(kind, int(m["heads"]), int(m.get("vdim") or m["dim"]), dim=int(m["dim"]),
                                         kv_heads=int(m.get("kv_heads") or m["heads"]), scale=float(m["scale"]),
                                         temp_coef=float(qt.get("coef") or 0.0), temp_every=int(qt.get("every") or 0),
                                         bias_max=int(m["bias_max"]), kv_from=-1 if src is None else int(src)))
            elif kind == "mamba2":
                hp.mixers.append(MixSpec(kind, int(m["heads"]), int(m["vdim"]), state=int(m["state"]),
                                         groups=int(m.get("groups") or 1), taps=int(m["conv"]),
                                         norm_groups=int(m.get("norm_groups") or 1)))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            f = L.get("mlp")
            if not f:
                hp.mlps.append(None)
            elif f.get("kind") == "dense":
                hp.mlps.append(FfSpec("dense", int(f["ff"])))
            elif f.get("kind") == "moe":
                sh = f.get("shared") or {}
                hp.mlps.append(FfSpec("moe", int(f["expert"]["ff"]), float(f["expert"]["limit"]),
                                      int(f["router"]["experts"]), int(f["router"]["top"]),
                                      int(sh.get("ff") or 0), float(sh.get("limit") or 0.0)))
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
        for i, m in enumerate(hp.mixers):
            if m.kind != "attention" or m.kv_from < 0:
                continue
            o = hp.mixers[m.kv_from] if 0 <= m.kv_from < i else None
            if o is None or o.kind != "attention" or o.kv_from >= 0:
                raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with projections of its own")
            if (o.kv_heads, o.dim, o.vdim) != (m.kv_heads, m.dim, m.vdim):
                raise ValueError(f"layer {i}: kv_from layer {m.kv_from} has other key / value shapes")
        return hp


@dataclass
class _Expert:
    gate_up: ops.QWeight
    down: ops.QWeight


@dataclass
class _Layer:
    norm1: torch.Tensor
    win: ops.QWeight                   # attention: q | k | v rows (q only with kv_from); mamba2: the input projection
    wo: ops.QWeight
    norm2: Optional[torch.Tensor] = None
    bias: Optional[torch.Tensor] = None          # attention: distance-bias table fp32 [bias_max + 1, H]
    sink: Optional[torch.Tensor] = None          # fp32 [H]
    conv: Optional[torch.Tensor] = None          # mamba2: fp32 [C, taps]
    conv_t: Optional[torch.Tensor] = None        # the same tap-major, [taps, C] (the vectorised kernel's layout)
    conv_b: Optional[torch.Tensor] = None
    dt_bias: Optional[torch.Tensor] = None
    a_log: Optional[torch.Tensor] = None
    d_skip: Optional[torch.Tensor] = None
    mix_norm: Optional[torch.Tensor] = None
    gate_up: Optional[ops.QWeight] = None        # dense feed-forward
    down: Optional[ops.QWeight] = None
    router: Optional[torch.Tensor] = None        # fp32 [E, D]
    router_b: Optional[torch.Tensor] = None
    wg: Optional[torch.Tensor] = None            # stacked expert weights [E, F, D] / [E, D, F], activation dtype
    wu: Optional[torch.Tensor] = None
    wd: Optional[torch.Tensor] = None
    experts: Optional[List[_Expert]] = None
    moe_gu: Optional[object] = None              # ops.MoEWeights where the grouped expert GEMMs take the shape
    moe_down: Optional[object] = None
    shared: Optional[_Expert] = None
    side_gate: Optional[ops.QWeight] = None
    side_proj: Optional[ops.QWeight] = None
    side_norm: Optional[torch.Tensor] = None


class VinozenModel:
    # what this family launches from ops/csrc (ops.require_kernels: a first run compiles only these)
    kernel_sources = ("elementwise.hip", "norm_chain.hip", "rope_pages.hip", "retention.hip", "mamba2.hip",
                      "attention_mix.hip", "attention.hip", "moe_dense.hip", "moe.hip", "sampling.hip", "decode_loop.hip",
                      "gemm_skinny.hip")
    stateful = True         # convolution tails and recurrent state per sequence: state slots, no prefix-cache reuse
    mixed_batches = True    # prompt portions and decode rows of different sequences in one forward

    def __init__(self, reader, device: torch.device, tp: Optional[TPInfo] = None, max_pos: Optional[int] = None,
                 rope_overrides: Optional[dict] = None, lora=None, dtype: torch.dtype = torch.bfloat16):
        self.tp = tp or TPInfo()
        if self.tp.world > 1:
            raise ValueError("vinozen: tensor parallelism is not implemented for this design")
        if lora is not None:
            raise ValueError("vinozen: LoRA adapters are not supported")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("vinozen: serving dtype is bfloat16 or float32")
        self.device, self.dtype = device, dtype
        self.f32 = dtype == torch.float32
        self.hp = hp = VinozenHParams.from_config(reader.config, str(reader.kv.get("general.name", "")))
        self.max_pos = max_pos or 1 << 20
        self.vocab_local = hp.n_vocab
        self.T = reader.tensors
        D = hp.n_embd
        f32, qw, sh = self._f32, self._qw, self._shaped
        emb = sh("embed", (hp.n_vocab, D))
        self.tok_embd = ops.QWeight.from_float(emb.to(device))      # bf16 table, exact: stored as bf16
        self.output = qw(emb)                                       # the table is also the head (unscaled)
        self.pos_freqs = ops.sinusoid_freqs(D, 10000.0, device)
        self.side_table = None
        if hp.side_dim:
            self.side_table = sh("side.embed", (hp.n_vocab, hp.n_layer * hp.side_dim)).to(device=device, dtype=torch.bfloat16).contiguous()
        self.layers: List[_Layer] = []
        for i, (m, f) in enumerate(zip(hp.mixers, hp.mlps)):
            p = f"l{i}."
            L = self._load_attention(p, m) if m.kind == "attention" else self._load_mamba2(p, m)
            if f is not None:
                L.norm2 = f32(p + "norm2", (D,))
                self._load_ff(L, p + "mlp.", f)
            if hp.side_dim:
                L.side_gate = qw(sh(p + "side.gate", (hp.side_dim, D)))
                L.side_proj = qw(sh(p + "side.proj", (D, hp.side_dim)))
                L.side_norm = f32(p + "side.norm", (D,))
            self.layers.append(L)
        self.out_norm = ("ln", f32("final.norm", (D,)), hp.norm_eps)
        self._aranges: Dict[int, tuple] = {}
        self.T = None

    # --------------------------------------------------------------------------- loading
    def _raw(self, name: str) -> torch.Tensor:
        if name not in self.T:
            raise KeyError(f"vinozen: missing tensor {name}")
        t = self.T[name]
        return torch.from_numpy(dequantize(t.data, t.ggml_type, t.shape).astype(np.float32).reshape(t.shape))

    def _shaped(self, name: str, shape) -> torch.Tensor:
        w = self._raw(name)
        if tuple(w.shape) != tuple(shape):
            raise ValueError(f"vinozen: {name} is {tuple(w.shape)}, the config asks for {tuple(shape)}")
        return w

    def _f32(self, name: str, shape) -> torch.Tensor:
        return self._shaped(name, shape).to(self.device).contiguous()

    def _qw(self, w: torch.Tensor) -> ops.QWeight:
        w = w.to(self.device)
        return ops.QWeight.from_f32(w) if self.f32 else ops.QWeight.from_float(w)

    def _load_attention(self, p: str, m: MixSpec) -> _Layer:
        D, H = self.hp.n_embd, m.heads
        sh = self._shaped
        if H % m.kv_heads:
            raise ValueError(f"{p}: heads must be a multiple of kv_heads")
        rows = [sh(p + "mix.q", (H * m.dim, D))]
        if m.kv_from < 0:
            rows += [sh(p + "mix.k", (m.kv_heads * m.dim, D)), sh(p + "mix.v", (m.kv_heads * m.vdim, D))]
        L = _Layer(self._f32(p + "norm1", (D,)), self._qw(torch.cat(rows, 0)), self._qw(sh(p + "mix.o", (D, H * m.vdim))))
        rel = self._raw(p + "mix.rel")
        if rel.dim() != 2 or rel.shape[1] != H:
            raise ValueError(f"{p}mix.rel: one column per head")
        L.bias = ops.bucketed_bias(rel, m.bias_max).to(self.device)
        L.sink = self._f32(p + "mix.sink", (H,))
        return L

    def _load_mamba2(self, p: str, m: MixSpec) -> _Layer:
        D, H = self.hp.n_embd, m.heads
        sh = self._shaped
        inner, GN = H * m.vdim, m.groups * m.state
        if H % m.groups or inner % m.norm_groups:
            raise ValueError(f"{p}: heads must be a multiple of groups, heads * vdim of norm_groups")
        C = inner + 2 * GN
        L = _Layer(self._f32(p + "norm1", (D,)), self._qw(sh(p + "mix.in", (2 * inner + 2 * GN + H, D))),
                   self._qw(sh(p + "mix.o", (D, inner))))
        L.conv = self._f32(p + "mix.conv", (C, m.taps))
        L.conv_t = L.conv.t().contiguous()
        L.conv_b = self._f32(p + "mix.conv.b", (C,))
        L.dt_bias, L.a_log, L.d_skip = (self._f32(p + n, (H,)) for n in ("mix.dt_bias", "mix.A_log", "mix.D"))
        L.mix_norm = self._f32(p + "mix.norm", (inner,))
        return L

    def _expert(self, p: str, ff: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        D = self.hp.n_embd
        return (self._shaped(p + "gate", (ff, D)), self._shaped(p + "up", (ff, D)), self._shaped(p + "down", (D, ff)))

    def _load_ff(self, L: _Layer, p: str, f: FfSpec) -> None:
        D, qw = self.hp.n_embd, self._qw
        if f.kind == "dense":
            g, u, d = self._expert(p, f.ff)
            L.gate_up, L.down = qw(torch.cat([g, u], 0)), qw(d)
            return
        if not 1 <= f.top <= f.experts:
            raise ValueError(f"{p}: top must lie in 1 .. experts")
        L.router = self._f32(p + "router", (f.experts, D))
        L.router_b = self._f32(p + "router.b", (f.experts,)) if p + "router.b" in self.T else None
        ws = [self._expert(p + f"e{e}.", f.ff) for e in range(f.experts)]
        L.wg, L.wu, L.wd = (torch.stack([w[k] for w in ws]).to(device=self.device, dtype=self.dtype).contiguous()
                            for k in range(3))
        L.experts = [_Expert(qw(torch.cat([g, u], 0)), qw(d)) for g, u, d in ws]
        if not self.f32 and self.device.type == "cuda" and D % 256 == 0 and f.ff % 256 == 0:
            # the framework's grouped expert GEMMs (one weight stream per active expert, device
            # routing, no host sync) read [gate; up] fused per expert
            L.moe_gu = ops.MoEWeights([e.gate_up for e in L.experts])
            L.moe_down = ops.MoEWeights([e.down for e in L.experts])
        if f.shared_ff:
            g, u, d = self._expert(p + "shared.", f.shared_ff)
            L.shared = _Expert(qw(torch.cat([g, u], 0)), qw(d))

    # --------------------------------------------------------------------------- engine interface
    def _specs(self):
        """KVCache.layered spec of every layer: pages for attention layers with projections of their
        own, (convolution tail, recurrent state) for mamba2 layers."""
        out = []
        for m in self.hp.mixers:
            if m.kind == "attention":
                out.append((m.kv_heads, m.dim, m.vdim, None) if m.kv_from < 0 else (0, 0, 0, None))
            else:
                C = m.heads * m.vdim + 2 * m.groups * m.state
                out.append((0, 0, 0, [((max(m.taps - 1, 0), C), None), ((m.heads, m.vdim, m.state), torch.float32)]))
        return out

    def kv_bytes_per_token(self) -> int:
        es = 4 if self.f32 else 2
        return max(es, sum(g * (dk + dv) * es for g, dk, dv, *_ in self._specs()))

    def new_kv_cache(self, num_blocks: int, block_size: int, state_slots: int = 0) -> KVCache:
        return KVCache.layered(self._specs(), num_blocks, block_size, self.device, self.dtype, state_slots)

    def decode_workspace(self, Bp: int, ctx: int, block_size: int):
        """Split-KV buffers of the decode attention kernel per (heads, kv heads, width) of the layers it serves."""
        out = {}
        for m in self.hp.mixers:
            if m.kind == "attention" and self._decode_kernel_ok(m, block_size):
                key = (m.heads, m.kv_heads, m.dim)
                if key not in out:
                    out[key] = ops.decode_workspace(Bp, m.heads, m.kv_heads, m.dim, ctx, self.device, block_size)
        return out or None

    def _decode_kernel_ok(self, m: MixSpec, block_size: int) -> bool:
        """Decode batches of this layer on the framework's split-KV decode attention kernel (the llama
        families'): bf16, equal key and value widths it is instantiated for; it takes the bias table and the sink."""
        return (not self.f32 and self.device.type == "cuda" and m.dim == m.vdim and m.dim in (64, 80, 96, 128, 192, 256)
                and m.heads // m.kv_heads <= 16 and block_size % 16 == 0 and (128 % block_size == 0 or block_size % 128 == 0)
                and ops._has("la_attn_decode"))

    def prefill_tiles(self, q_lens, device):
        """((16-row work tiles of the leading prompt portions for ops.attn_mix, 64-row tiles of the same
        portions for ops.attn_prefill where a layer has the widths that kernel takes), rows they cover)."""
        if device.type != "cuda" or self.f32:
            return None, 0
        mix, rows = ops.attn_mix_tiles(q_lens, device)
        pf = None
        if any(m.kind == "attention" and self._prefill_kernel_ok(m) for m in self.hp.mixers):
            pf = ops.prefill_tiles(q_lens, device)
        return (mix, pf), rows

    def _prefill_kernel_ok(self, m: MixSpec) -> bool:
        """Batches of prompt portions only, for this layer, on the framework's prefill attention kernel (the
        llama families': 64 query rows of one head per workgroup): bf16, equal key and value widths it is
        instantiated for; it takes the bias table and the sink."""
        return (not self.f32 and self.device.type == "cuda" and m.dim == m.vdim and m.dim in (64, 80, 96, 128, 192, 256)
                and ops._has("la_attn_prefill"))

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

    def _unit(self, x: torch.Tensor, e: _Expert, ff: int, limit: float):
        """One clamped gated expert on rows x: down(glu_clamp(gate|up x))."""
        return ops.linear(ops.glu_clamp(ops.linear(x, e.gate_up), ff, limit, out_dtype=self.dtype), e.down)

    def _routed(self, L: _Layer, f: FfSpec, xn: torch.Tensor) -> torch.Tensor:
        """fp32 [T, D]: the weighted sum of every row's chosen experts."""
        T = xn.shape[0]
        ids, wts = ops.router_softmax(xn, L.router, L.router_b, f.top)
        capturing = xn.is_cuda and torch.cuda.is_current_stream_capturing()
        if L.moe_gu is not None and (T < MOE_DENSE_MIN_T or capturing) and T > 2:
            # grouped expert GEMMs on the routed rows, as the Mixtral path: gate|up, the clamped unit,
            # then the down projection with the routing weights
            order, off = ops.moe_route(ids, f.experts)
            gu = ops.moe_linear(xn, L.moe_gu, order, off, f.top, T)
            h = ops.glu_clamp(gu, f.ff, f.limit, out_dtype=self.dtype)
            return ops.moe_linear(h, L.moe_down, order, off, f.top, T, down=True, wts=wts).dense()
        if T <= MOE_PAIR_MAX_T or capturing:
            return ops.moe_pairs(xn, L.wg, L.wu, L.wd, ids, wts, clamp=(f.limit, 1.702))
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
                y = self._dense(self._unit(xs[r0:r1].contiguous(), L.experts[e], f.ff, f.limit)).float()
                out.index_add_(0, tok[r0:r1], y * wsel[r0:r1].unsqueeze(1))
        return out

    def _mlp(self, L: _Layer, f: FfSpec, xn: torch.Tensor):
        if f.kind == "dense":
            gu = ops.linear(xn, L.gate_up)
            if not self.f32 and (f.ff % 4 == 0 or not xn.is_cuda):
                h = ops.act(gu, f.ff, ops.ACT_SWIGLU)
            else:
                x = self._dense(gu).float()
                h = (torch.nn.functional.silu(x[:, :f.ff]) * x[:, f.ff:]).to(self.dtype)
            return ops.linear(h, L.down)
        y = self._routed(L, f, xn)
        if L.shared is not None:
            y = y + self._dense(self._unit(xn, L.shared, f.shared_ff, f.shared_limit)).float()
        return y

    def _attention(self, L: _Layer, m: MixSpec, i: int, xn, fb, kv, row_seq, cu_q, tiles, tile_rows, splits, ws=None):
        proj = self._dense(ops.linear(xn, L.win))
        own = m.kv_from < 0
        src = i if own else m.kv_from
        q = ops.qk_norm_pages(proj, m.heads, m.dim, m.kv_heads if own else 0, m.dim, m.vdim, fb.pos, fb.slots,
                              self.hp.norm_eps, m.temp_coef, m.temp_every, kv.k[src] if own else None,
                              kv.v[src] if own else None)
        if fb.decode and fb.seq_lens is not None and self._decode_kernel_ok(m, kv.block_size):
            T = q.shape[0]
            return ops.attn_decode(q.view(T, m.heads, m.dim), kv.k[src], kv.v[src], fb.block_tables, fb.seq_lens, m.scale,
                                   fb.max_len, workspace=ws, dist_bias=L.bias, sink=L.sink).view(T, m.heads * m.vdim)
        if isinstance(tiles, tuple):
            tiles, pf = tiles
            if (pf is not None and not fb.decode and tile_rows == q.shape[0] and fb.ctx_lens is not None
                    and self._prefill_kernel_ok(m) and kv.block_size % 16 == 0):
                T = q.shape[0]
                return ops.attn_prefill(q.view(T, m.heads, m.dim), kv.k[src], kv.v[src], cu_q, fb.ctx_lens, fb.block_tables,
                                        m.scale, tiles=pf, dist_bias=L.bias, sink=L.sink).view(T, m.heads * m.vdim)
        return ops.attn_mix(q, kv.k[src], kv.v[src], row_seq, fb.pos, fb.block_tables, m.heads, m.scale,
                            tiles=tiles, tile_rows=tile_rows, cu_q=cu_q, key_splits=splits, dist_bias=L.bias, sink=L.sink)

    def _mamba2(self, L: _Layer, m: MixSpec, i: int, xn, fb, kv, cu_q):
        proj = self._dense(ops.linear(xn, L.win))            # [T, z | x | B | C | dt]
        conv_state, ssm_state = kv.state[i]
        return ops.mamba2(proj, m.heads, m.vdim, m.state, m.groups, L.conv, L.conv_b, L.dt_bias, L.a_log, L.d_skip,
                          L.mix_norm, m.norm_groups, self.hp.norm_eps, fb.pos, cu_q, fb.sslots, conv_state, ssm_state,
                          max_rows=1 if fb.decode else fb.max_q, conv_wt=L.conv_t)

    def forward(self, fb: ForwardBatch, kv: KVCache, attn_workspace=None, return_hidden: bool = False,
                local_logits: bool = False, layer_out: Optional[list] = None) -> torch.Tensor:
        """fp32 logits [R, V] of the rows fb.logits_idx selects (all rows when None).  Rows of one
        sequence are consecutive; fb.decode batches bring one row per sequence (fb.sslots per row),
        other batches fb.cu_q / fb.row_seq / fb.sslots per sequence.  layer_out: a list that
        receives the fp32 residual stream after every layer (diagnostics)."""
        hp = self.hp
        T = fb.tokens.shape[0]
        if fb.sslots is None or (kv.state is None and any(m.kind == "mamba2" for m in hp.mixers)):
            raise ValueError("vinozen: the batch needs state slots (engine built without a state pool?)")
        if fb.decode:
            row_seq, cu_q, tiles = self._single_rows(T)
            tile_rows = T if (DECODE_TILES and not self.f32 and fb.tokens.is_cuda) else 0
            splits = max(1, min(32, DECODE_WGS // max(T, 1), -(-(fb.max_len or 1) // 32)))
        else:
            row_seq, cu_q, tiles, tile_rows = fb.row_seq, fb.cu_q, fb.tiles, fb.tile_rows
            if row_seq is None:
                raise ValueError("vinozen: prompt batches need fb.row_seq")
            splits = 1
        if fb.tokens.is_cuda and hp.n_embd % 8:   # the embedding kernel reads 8 columns per thread
            res = self.tok_embd.materialize_bf16().index_select(0, fb.tokens.long()).float() * hp.embed_scale
        else:
            res = ops.embed(fb.tokens, self.tok_embd, hp.embed_scale)
        if not res.is_contiguous() or res.dtype != torch.float32:
            res = res.float().contiguous()
        ops.sinusoid_add(res, fb.pos, self.pos_freqs)
        nc = lambda branch, post, pre: ops.norm_chain(res, branch, post, pre, out_dtype=self.dtype)  # noqa: E731
        eps, n = hp.norm_eps, hp.n_layer
        cast = ("cast",)
        xn = nc(None, None, cast)        # the sublayers read the stream itself
        for i, (L, m, f) in enumerate(zip(self.layers, hp.mixers, hp.mlps)):
            if m.kind == "attention":
                ws = attn_workspace.get((m.heads, m.kv_heads, m.dim)) if isinstance(attn_workspace, dict) else None
                a = self._attention(L, m, i, xn, fb, kv, row_seq, cu_q, tiles, tile_rows, splits, ws)
            else:
                a = self._mamba2(L, m, i, xn, fb, kv, cu_q)
            last = self.out_norm if i + 1 == n else cast       # what the layer's last boundary hands on
            o = ops.linear(a, L.wo)
            xn = nc(o, ("ln", L.norm1, eps), cast if (f is not None or L.side_gate is not None) else last)
            if f is not None:
                xn = nc(self._mlp(L, f, xn), ("ln", L.norm2, eps), cast if L.side_gate is not None else last)
            if L.side_gate is not None:
                g = ops.side_gate(ops.linear(xn, L.side_gate), fb.tokens, self.side_table, i * hp.side_dim, self.dtype)
                xn = nc(ops.linear(g, L.side_proj), ("rms", L.side_norm, eps), last)
            if layer_out is not None:
                layer_out.append(res.clone())
        if return_hidden:
            return xn
        rows = xn if fb.logits_idx is None else xn.index_select(0, fb.logits_idx)
        lp = ops.linear(rows.contiguous(), self.output)
        return lp.t[0] if (lp.t.dim() == 3 and lp.t.shape[0] == 1 and lp.t.dtype == torch.float32) else self._dense(lp).float()
