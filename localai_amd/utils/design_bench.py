"""Prefill and decode throughput of a model design beside the closest decoder family at equal
layer sizes (bench.py --design-compare): random weights, bf16, one GPU.

For each size two-layer models are built -- Suganex: dense feed-forwards (beside a llama
checkpoint) and routed experts (beside a Mixtral-style checkpoint); Dadizen: one model per mixer
kind (windowed attention, latent attention, retention) beside the llama checkpoint; Vinozen:
attention with a dense feed-forward, attention with routed experts, the state-space mixer, beside
the llama and Mixtral-style checkpoints; Gosuvik: the delta rule, latent attention with routed experts,
the parallel mixer, beside the same two -- all stored as
dense bf16 weights so every GEMM takes the same library path, and each is timed through its engine's own
batch construction (native scheduler, paged KV pool, state slots) and `model.forward`:
  prefill: `n_seq` prompts of `prompt` tokens in one batch, tokens/s;
  decode:  `batch` sequences holding `context` tokens each, one token per sequence and step, tokens/s
           (1536 by default: a Suganex row then sees the 513 keys of its chunk of 1024, a llama row all 1537).
The forward is repeated on the same batch (it rewrites the same K/V slots), so the numbers are the
kernels' and the GEMMs', without the host's planning time.
"""
from __future__ import annotations

import json
import os
import time
from typing import Dict, List

import numpy as np
import torch

SIZES = {
    # name: width, heads, kv heads, head width, dense ff, experts, top, expert ff, chunk
    "2k": dict(width=2048, heads=16, kv=4, dim=128, ff=8192, experts=8, top=2, eff=2048, chunk=1024),
    "tiny": dict(width=256, heads=4, kv=2, dim=64, ff=512, experts=4, top=2, eff=256, chunk=64),   # dry runs
    "4k": dict(width=4096, heads=32, kv=8, dim=128, ff=14336, experts=8, top=2, eff=3584, chunk=1024),
}
VOCAB = 32000


def _llama(size: str, cache: str, moe: bool = False) -> str:
    from ..models import synth
    s = SIZES[size]
    kind = "moe" if moe else "dense"
    g = os.path.join(cache, f"llama-{size}-{kind}-f16.gguf")
    if not os.path.exists(g):
        pre = synth.Preset(n_layer=2, n_embd=s["width"], n_head=s["heads"], n_head_kv=s["kv"], head_dim=s["dim"],
                           n_ff=s["eff"] if moe else s["ff"], n_vocab=VOCAB, ctx=8192, qtype="F16",
                           n_expert=s["experts"] if moe else 0, n_expert_used=s["top"] if moe else 0,
                           tokenizer="mistral", name=f"llama-{size}-{kind}")
        synth.write_model(g + ".partial", pre)
        os.replace(g + ".partial", g)
    return g


def _dadizen_models(size: str, cache: str) -> Dict[str, str]:
    """Two equal layers of one mixer kind each: windowed attention (window = the size's chunk),
    latent attention (kv latent 4 head widths, rotated part half a head width, query latent 12 head
    widths: the proportions of the published latent-attention models), retention (half the heads
    at twice the value width, so the projections keep the attention layers' parameter count)."""
    from ..models import synth
    s = SIZES[size]
    out = {}
    for kind in ("attention", "latent_attention", "retention"):
        p = os.path.join(cache, f"dadizen-{size}-{kind}")
        if not os.path.exists(os.path.join(p, "model.safetensors")):
            kw = dict(heads=s["heads"], kv_heads=s["kv"], dim=s["dim"], vdim=s["dim"])
            if kind == "retention":
                kw = dict(heads=s["heads"] // 2, dim=s["dim"], vdim=2 * s["dim"])
            synth.write_dadizen(p, width=s["width"], kinds=(kind, kind), window=s["chunk"], rot_dim=s["dim"] // 2,
                                q_rank=min(12 * s["dim"], s["width"]), kv_rank=4 * s["dim"], ff=s["ff"],
                                side_dim=s["dim"], vocab=VOCAB, **kw)
        out[f"dadizen-{kind}"] = p
    out["llama-dense"] = _llama(size, cache)
    return out


def _vinozen_models(size: str, cache: str) -> Dict[str, str]:
    """Two equal layers each: attention with a dense feed-forward (beside the llama checkpoint), attention
    with routed experts and no shared expert (beside the Mixtral-style checkpoint, equal expert count
    and widths), the state-space mixer with a dense feed-forward (inner width twice the model width
    in heads of 64 channels, state 128, one group, 4 taps: the usual proportions of such layers)."""
    from ..models import synth
    s = SIZES[size]
    out = {}
    for kind in ("attention-dense", "attention-moe", "mamba2-dense"):
        p = os.path.join(cache, f"vinozen-{size}-{kind}")
        mix, f = kind.split("-")
        if not os.path.exists(os.path.join(p, "model.safetensors")):
            synth.write_vinozen(p, width=s["width"], kinds=(mix, mix), heads=s["heads"], kv_heads=s["kv"], dim=s["dim"],
                                vdim=s["dim"], m_heads=2 * s["width"] // 64, m_vdim=64, m_state=128, ff=s["ff"],
                                experts=s["experts"] if f == "moe" else 0, top=s["top"], expert_ff=s["eff"],
                                side_dim=s["dim"], vocab=VOCAB)
        out[f"vinozen-{kind}"] = p
    out["llama-dense"] = _llama(size, cache)
    out["mixtral-moe"] = _llama(size, cache, moe=True)
    return out


def _gosuvik_models(size: str, cache: str) -> Dict[str, str]:
    """Two equal layers each: the delta rule (as many q / k heads as heads, head width of the size, decay
    and gate projections of one head width, 4 taps) with the dense polynomial feed-forward; latent
    attention (latent 4 head widths, rotated part half a head width, window = the size's chunk) with
    routed experts; the parallel mixer (grouped-query sink attention of the size's heads, window = the
    size's chunk, beside a matrix memory of half as many heads) with the dense feed-forward."""
    from ..models import synth
    s = SIZES[size]
    out = {}
    for kind, moe in (("channel_delta", False), ("latent_attention", True), ("parallel", False)):
        p = os.path.join(cache, f"gosuvik-{size}-{kind}")
        if not os.path.exists(os.path.join(p, "model.safetensors")):
            kv = s["heads"] if kind == "channel_delta" else s["kv"]
            synth.write_gosuvik(p, width=s["width"], kinds=(kind, kind), heads=s["heads"], kv_heads=kv, dim=s["dim"],
                                vdim=s["dim"], conv=4, rank=s["dim"], rot_dim=s["dim"] // 2, kv_rank=4 * s["dim"],
                                window=s["chunk"], r_heads=max(1, s["heads"] // 2), r_dim=s["dim"], r_vdim=s["dim"], ff=s["ff"],
                                experts=s["experts"] if moe else 0, top=s["top"], expert_ff=s["eff"], groups=4, vocab=VOCAB)
        out[f"gosuvik-{kind}" + ("-moe" if moe else "-dense")] = p
    out["llama-dense"] = _llama(size, cache)
    out["mixtral-moe"] = _llama(size, cache, moe=True)
    return out


def _models(size: str, cache: str) -> Dict[str, str]:
    from ..models import synth
    s = SIZES[size]
    out = {}
    for kind in ("dense", "moe"):
        moe = kind == "moe"
        p = os.path.join(cache, f"suganex-{size}-{kind}")
        if not os.path.exists(os.path.join(p, "model.safetensors")):
            synth.write_suganex(p, width=s["width"], n_layer=2, heads=s["heads"], kv_heads=s["kv"], dim=s["dim"],
                                vdim=s["dim"], conv=4, chunk=s["chunk"], ff=s["ff"], experts=s["experts"] if moe else 0,
                                top=s["top"], expert_ff=s["eff"], vocab=VOCAB)
        out[f"suganex-{kind}"] = p
        g = os.path.join(cache, f"llama-{size}-{kind}-f16.gguf")
        if not os.path.exists(g):
            pre = synth.Preset(n_layer=2, n_embd=s["width"], n_head=s["heads"], n_head_kv=s["kv"], head_dim=s["dim"],
                               n_ff=s["eff"] if moe else s["ff"], n_vocab=VOCAB, ctx=8192, qtype="F16",
                               n_expert=s["experts"] if moe else 0, n_expert_used=s["top"] if moe else 0,
                               tokenizer="mistral", name=f"llama-{size}-{kind}")
            synth.write_model(g + ".partial", pre)
            os.replace(g + ".partial", g)
        out[("mixtral" if moe else "llama") + f"-{kind}"] = g
    return out


def DEVICE() -> str:
    return "cuda:0" if torch.cuda.is_available() else "cpu"


def _time(fn, iters: int) -> float:
    for _ in range(2):
        fn()
    if not torch.cuda.is_available():
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        return (time.perf_counter() - t0) / iters
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / 1e3 / iters


def _measure(path: str, n_seq: int, prompt: int, batch: int, context: int, iters: int) -> Dict[str, float]:
    from ..engine.llm_engine import EngineConfig, LLMEngine
    from ..models.decoder import DecoderModel, ForwardBatch
    tokens = max(n_seq * prompt, batch * (context + 32))
    eng = LLMEngine(EngineConfig(model_path=path, device=DEVICE(), context_size=max(prompt, context + 32) + 32,
                                 max_num_seqs=max(n_seq, batch), max_batched_tokens=n_seq * prompt, block_size=32,
                                 max_kv_tokens=tokens + 64 * max(n_seq, batch), prefix_cache=False, use_graphs=False,
                                 blas_tune=False))
    rng = np.random.default_rng(0)
    dm = isinstance(eng.model, DecoderModel)

    def batch_of(ids, n):
        for i in ids:
            if eng.sched.has(i):
                eng.sched.extend(i, rng.integers(0, VOCAB, size=n).tolist())
            else:
                eng.sched.add(i, rng.integers(0, VOCAB, size=n).tolist(), 0)
        plan = eng.sched.schedule_explicit([(i, n) for i in ids])
        k, q = len(ids), plan["p_qlen"]
        dec = bool(plan["p_decode"].all()) and n == 1
        fb = ForwardBatch(tokens=eng._dev(plan["p_tokens"]), pos=eng._dev(plan["p_pos"]), slots=eng._dev(plan["p_slots"]),
                          decode=dec, block_tables=eng._dev(plan["p_bt"]),
                          logits_idx=eng._dev(np.asarray(plan["p_cu"][1:] - 1, dtype=np.int64)))
        if dec:
            fb.seq_lens, fb.max_len = eng._dev(plan["p_ctx"]), int(plan["p_ctx"].max())
        else:
            fb.cu_q, fb.ctx_lens = eng._dev(plan["p_cu"]), eng._dev(plan["p_ctx"])
            if not dec:
                fb.tiles, fb.tile_rows = eng.model.prefill_tiles(q, eng.device)
        if not dm:
            fb.sslots = eng._dev(plan["p_sslot"])
            fb.row_seq = eng._dev(np.repeat(np.arange(k, dtype=np.int32), q))
            fb.max_q = int(max(q))
        return fb

    out = {}
    fb = batch_of(list(range(1, n_seq + 1)), prompt)
    t = _time(lambda: eng.model.forward(fb, eng.kv), iters)
    out["prefill_tok_s"] = n_seq * prompt / t
    out["prefill_ms"] = t * 1e3
    for i in range(1, n_seq + 1):
        eng.sched.finish(i)
    ids = list(range(100, 100 + batch))
    left = context
    while left > 0:   # fill the contexts in chunks that fit one batch
        n = min(left, max(1, (n_seq * prompt) // batch))
        eng.model.forward(batch_of(ids, n), eng.kv)
        left -= n
    fb = batch_of(ids, 1)
    t = _time(lambda: eng.model.forward(fb, eng.kv), iters * 4)
    out["decode_tok_s"] = batch / t
    out["decode_ms"] = t * 1e3
    del eng
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return out


def run(design: str, sizes: List[str], cache: str, n_seq: int = 4, prompt: int = 2048, batch: int = 64,
        context: int = 1536, iters: int = 5) -> dict:
    if design not in ("suganex", "dadizen", "vinozen", "gosuvik"):
        raise SystemExit(f"--design-compare: unknown design {design!r} (suganex, dadizen, vinozen, gosuvik)")
    os.makedirs(cache, exist_ok=True)
    res = {"design": design, "dtype": "bf16", "data": "synthetic", "layers": 2,
           "workload": {"prefill": f"{n_seq} x {prompt} tokens", "decode": f"batch {batch} at context {context}"},
           "sizes": {}}
    for size in sizes:
        t0 = time.time()
        paths = {"suganex": _models, "dadizen": _dadizen_models, "vinozen": _vinozen_models,
                 "gosuvik": _gosuvik_models}[design](size, cache)
        row = {}
        for name, p in paths.items():
            row[name] = {k: round(v, 3 if k.endswith("ms") else 1)
                         for k, v in _measure(p, n_seq, prompt, batch, context, iters).items()}
            print(f"# {size} {name}: {row[name]}", flush=True)
        res["sizes"][size] = dict(SIZES[size], **row)
        print(f"# {size} done in {time.time() - t0:.0f} s", flush=True)
    print(json.dumps(res), flush=True)
    return res
