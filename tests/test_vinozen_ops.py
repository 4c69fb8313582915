"""The Vinozen mechanisms one by one -- operator layer (PyTorch CPU paths, HIP kernels under `gpu`)
against the plain functions of tests/vinozen_oracle.py -- with inputs made so that a fault shows:
a bias bucket that towers over the others, seen from just inside and just outside its distances; a
(query, key) pair pointing the same way far back and at page borders; sinks that swallow a head or
vanish; temperature steps at the positions where they change; state slots and pages holding another
sequence's leftovers; a decay that forgets nothing."""
import math

import numpy as np
import pytest
import torch

import vinozen_oracle as oracle
from localai_amd import ops

MODES = [("cpu", torch.float32), ("cpu", torch.bfloat16),
         pytest.param("cuda:0", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda:0", torch.bfloat16, marks=pytest.mark.gpu)]
F64 = torch.float64


def i32(x, dev):
    return torch.tensor(np.asarray(x), dtype=torch.int32, device=dev)


def rel(got, want):
    want = want.float()
    return float((got.float().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-6))


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


def rounded(x, dtype):
    """Test inputs as the operator sees them: representable in its dtype."""
    return x.to(dtype).float()


# --------------------------------------------------------------------------------------- norms, positions
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("D", [40, 37])
def test_layer_norm_after_the_branch_and_before_the_head(device, dtype, D):
    g = torch.Generator().manual_seed(D)
    T = 7
    res0 = torch.randn(T, D, generator=g) * 3
    br = rounded(torch.randn(T, D, generator=g) * 2 + 1.5, dtype)        # a mean far from zero
    w1, w2 = 1 + 0.3 * torch.randn(D, generator=g), torch.randn(D, generator=g)
    res = res0.clone().to(device)
    out = ops.norm_chain(res, br.to(device=device, dtype=dtype), ("ln", w1.to(device), 1e-3), ("cast",), out_dtype=dtype)
    want = res0 + oracle.layer_norm(br.double(), w1.double(), 1e-3)
    assert rel(res, want) < 2e-6 and rel(out, want) < tol(dtype)
    # fp32 split-K slabs in, the model's norm of the updated stream out
    res = res0.clone().to(device)
    slabs = torch.stack([br * 0.5, br * 0.25, br * 0.25]).to(device)
    out = ops.norm_chain(res, ops.Partial(slabs), ("ln", w1.to(device), 1e-5), ("ln", w2.to(device), 1e-2), out_dtype=dtype)
    want = res0 + oracle.layer_norm(br.double(), w1.double(), 1e-5)
    assert rel(res, want) < 2e-6 and rel(out, oracle.layer_norm(want, w2.double(), 1e-2)) < tol(dtype)
    # the stream only read
    out = ops.norm_chain(res, None, None, ("ln", w2.to(device), 1e-6), out_dtype=dtype)
    assert rel(out, oracle.layer_norm(want, w2.double(), 1e-6)) < tol(dtype)


@pytest.mark.parametrize("device", ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("D", [16, 37])
def test_sinusoid_positions_even_and_odd_widths(device, D):
    pos = [0, 1, 2, 63, 64, 1000, 4095]
    res = torch.zeros(len(pos), D, device=device)
    ops.sinusoid_add(res, i32(pos, device), ops.sinusoid_freqs(D, 10000.0, device))
    want = torch.stack([oracle.sinusoid(p, D) for p in pos])
    assert float((res.cpu().double() - want).abs().max()) < 5e-4        # fp32 angles of a few thousand radians
    assert float((res.cpu().double() - want)[:5].abs().max()) < 1e-5


@pytest.mark.parametrize("B,far", [(8, 20), (7, 33), (32, 100), (4, 5), (6, 9)])
def test_bias_table_follows_the_buckets(B, far):
    relt = torch.arange(B * 3, dtype=torch.float32).view(B, 3)
    tab = ops.bucketed_bias(relt, far)
    assert tuple(tab.shape) == (far + 1, 3)
    for n in range(far + 1):
        assert float(tab[n, 0]) == float(relt[oracle.bucket(n, B, far), 0]), n
    assert float(tab[far, 1]) == float(relt[B - 1, 1])                   # from `far` on: the last bucket
    assert oracle.bucket(far * 7, B, far) == B - 1
    assert [oracle.bucket(n, B, far) for n in range(B // 2)] == list(range(B // 2))


# --------------------------------------------------------------------------------------- unit-norm q / k, temperature
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("H,G,Dk,Dv,every", [(4, 2, 10, 6, 7), (3, 3, 64, 16, 1), (2, 1, 33, 8, 0)])
def test_unit_norm_queries_keys_temperature_and_page_append(device, dtype, H, G, Dk, Dv, every):
    g = torch.Generator().manual_seed(H + Dk)
    BS, n = 8, 30
    pos = list(range(3, 3 + n))                     # crosses multiples of `every` and page borders
    C = H * Dk + G * Dk + G * Dv
    rows = rounded(torch.randn(n, C + 5, generator=g) * 3, dtype)       # a wider row: the op reads its first C columns
    m = {"heads": H, "kv_heads": G, "dim": Dk, "vdim": Dv, "q_temp": {"coef": 0.6, "every": every}}
    eye = torch.eye(C + 5, dtype=F64)
    W = {"q": eye[:H * Dk], "k": eye[H * Dk:H * Dk + G * Dk], "v": eye[H * Dk + G * Dk:C]}
    q_all, k_w, v_w = oracle.attention_qkv(W, "", m, torch.cat([torch.zeros(3, C + 5, dtype=F64), rows.double()]), 1e-4)
    q_w, k_w, v_w = q_all[3:], k_w[3:], v_w[3:]
    nb = 6
    kc = torch.full((nb, G, BS, Dk), 50.0, dtype=dtype, device=device)
    vc = torch.full((nb, G, BS // 8, Dv, 8), 50.0, dtype=dtype, device=device)
    slots = [8 * 4 + 5 + t if t < 3 else 8 * 1 + (t - 3) if t < 11 else 8 * 3 + (t - 11) if t < 19 else -1 for t in range(n)]
    q = ops.qk_norm_pages(rows.to(device=device, dtype=dtype), H, Dk, G, Dk, Dv, i32(pos, device), i32(slots, device), 1e-4,
                          0.6, every, kc, vc)
    assert rel(q, q_w.reshape(n, -1)) < tol(dtype)
    for t, s in enumerate(slots):
        if s >= 0:
            assert rel(kc[s // BS, :, s % BS], k_w[t]) < tol(dtype)
            assert rel(vc[s // BS, :, (s % BS) // 8, :, s % 8], v_w[t]) < tol(dtype)
    assert float(kc[0].float().min()) == 50.0 and float(kc[5].float().min()) == 50.0       # rows without a slot go nowhere
    # queries only (a layer that attends over another layer's pages)
    q2 = ops.qk_norm_pages(rows[:, :H * Dk].contiguous().to(device=device, dtype=dtype), H, Dk, 0, 0, 0, i32(pos, device), None,
                           1e-4, 0.6, every)
    assert rel(q2, q_w.reshape(n, -1)) < tol(dtype)
    if every:   # the step itself: position every - 1 is the first with floor((p + 1) / every) = 1
        assert oracle.temperature(every - 2, 0.6, every) == 1.0 or every == 1
        assert abs(oracle.temperature(every - 1, 0.6, every) - (1 + 0.6 * math.log(2))) < 1e-12


# --------------------------------------------------------------------------------------- attention: bias, sink, far keys
def _attn_case(device, dtype, H, G, Dk, Dv, BS, n, B, far, hot, sinks, towers, tiles, scale=1.0, every=0):
    """qk_norm_pages + attn_mix over shuffled pages, a prompt portion then single rows, against the
    oracle.  hot: a bucket of head 0's bias table that towers over the others; sinks: per head;
    towers: [(query position, key position)] pointing the same way (head 1 / its kv head)."""
    g = torch.Generator().manual_seed(n + B)
    rng = np.random.default_rng(B)
    C = H * Dk + G * Dk + G * Dv
    rows = torch.randn(n, C, generator=g) * 0.5
    g1 = 1 // (H // G)                                           # kv head of query head 1
    for p, (qi, kj) in enumerate(towers):
        d = p % Dk
        rows[qi, Dk:2 * Dk] = 0.01 * torch.randn(Dk, generator=g)
        rows[qi, Dk + d] = 9.0
        rows[kj, H * Dk + g1 * Dk:H * Dk + (g1 + 1) * Dk] = 0.01 * torch.randn(Dk, generator=g)
        rows[kj, H * Dk + g1 * Dk + d] = 9.0
    rows = rounded(rows, dtype)
    relt = torch.randn(B, H, generator=g) * 0.5
    if hot is not None:
        relt[hot, 0] = 14.0
    relt = rounded(relt, torch.bfloat16)
    sink = torch.tensor(sinks, dtype=torch.float32)
    eye = torch.eye(C, dtype=F64)
    W = {"q": eye[:H * Dk], "k": eye[H * Dk:H * Dk + G * Dk], "v": eye[H * Dk + G * Dk:]}
    m = {"heads": H, "kv_heads": G, "dim": Dk, "vdim": Dv, "q_temp": {"coef": 0.4, "every": every}}
    qw, kw_, vw = oracle.attention_qkv(W, "", m, rows.double(), 1e-5)
    want = oracle.attention_core(qw, kw_, vw, relt.double(), sink.double(), scale, far)
    nb = -(-n // BS)
    table = rng.permutation(nb + 3)[:nb]
    slots = np.array([int(table[t // BS]) * BS + t % BS for t in range(n)])
    kc = torch.full((nb + 3, G, BS, Dk), 50.0, dtype=dtype, device=device)      # leftovers everywhere
    vc = torch.full((nb + 3, G, BS // 8, Dv, 8), 50.0, dtype=dtype, device=device)
    bias = ops.bucketed_bias(relt, far).to(device)
    bt = i32([table], device)
    got = torch.zeros(n, H * Dv)
    cut = n - 20                                                 # a portion, then 20 single rows
    for a, b in [(0, cut)] + [(t, t + 1) for t in range(cut, n)]:
        pos = i32(np.arange(a, b), device)
        q = ops.qk_norm_pages(rows[a:b].to(device=device, dtype=dtype), H, Dk, G, Dk, Dv, pos, i32(slots[a:b], device), 1e-5,
                              0.4, every, kc, vc)
        kw = {}
        if tiles and device != "cpu":
            tl, tr = ops.attn_mix_tiles([b - a], device)
            kw = dict(tiles=tl, tile_rows=tr, cu_q=i32([0, b - a], device), key_splits=1 if b - a > 1 else 3)
        out = ops.attn_mix(q, kc, vc, i32(np.zeros(b - a), device), pos, bt, H, scale, dist_bias=bias,
                           sink=sink.to(device), **kw)
        got[a:b] = out.float().cpu()
    assert rel(got, want) < (1e-4 if dtype == torch.float32 else 3e-2)
    return got, want, rows


@pytest.mark.parametrize("device,dtype", MODES)
def test_a_towering_bucket_seen_from_its_edges_in_prompts_and_decoding(device, dtype):
    # 10 buckets, 5 exact and 5 logarithmic up to distance 40: bucket 7 covers distances 12 .. 17 here.  With
    # head 0's bias of that bucket far above the rest (and a small score scale), head 0's output is the mean of the values at those
    # distances: rows at 11 (none yet), 12 (one), 17 / 18 (the oldest enters and leaves), in the portion and decoded
    B, far, hot = 10, 40, 7
    dists = [n for n in range(200) if oracle.bucket(n, B, far) == hot]
    assert dists == list(range(dists[0], dists[-1] + 1)) and len(dists) > 2
    n, Dv = 70, 6
    got, want, rows = _attn_case(device, dtype, H=4, G=2, Dk=10, Dv=Dv, BS=8, n=n, B=B, far=far, hot=hot,
                                 sinks=[0.0, 0.5, -1.0, 2.0], towers=[], tiles=False, scale=0.01)
    v = rows[:, 4 * 10 + 2 * 10:4 * 10 + 2 * 10 + Dv]
    for t in (dists[0], dists[-1], dists[-1] + 1, 40, 49, 50, 55, 69):       # 50 on: decoded alone
        keys = [t - d for d in dists if t - d >= 0]
        assert float((got[t, :Dv] - v[keys].mean(0)).abs().max()) < 0.05, t


@pytest.mark.parametrize("device,dtype", MODES)
def test_far_keys_page_borders_and_sinks(device, dtype):
    # head 1's query at 270 / 285 / 290 / 299 points the way of one key hundreds of rows back (position 0,
    # the last slot of a page, the first of the next): its output is that key's value.  Head 0's sink
    # swallows the head (output near zero); head 2's is so low that it changes nothing
    H, G, Dk, Dv = 3, 1, 32, 8          # unit-normed: a matching pair scores scale * 32, any other key under half of it
    towers = [(270, 0), (285, 15), (290, 16), (299, 31)]
    got, want, rows = _attn_case(device, dtype, H=H, G=G, Dk=Dk, Dv=Dv, BS=16, n=300, B=6, far=64, hot=None,
                                 sinks=[90.0, -2.0, -60.0], towers=towers, tiles=False, scale=1.5, every=128)
    v = rows[:, H * Dk + G * Dk:]
    for qi, kj in towers:
        assert float((got[qi, Dv:2 * Dv] - v[kj]).abs().max()) < 0.05, (qi, kj)
    assert float(got[:, :Dv].abs().max()) < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("B,far,hot", [(16, 50, 11), (9, 33, 6)])
def test_bucket_edges_and_sinks_on_the_matrix_core_tiles(B, far, hot):
    # widths the tile kernel takes (bf16, key width % 32, value width % 16): the same edges, portion rows on
    # 16-row tiles, single rows on one-row tiles split over the keys (the sink counted by one split only)
    dists = [n for n in range(300) if oracle.bucket(n, B, far) == hot]
    n, Dv = 120, 32
    got, want, rows = _attn_case("cuda:0", torch.bfloat16, H=4, G=2, Dk=64, Dv=Dv, BS=16, n=n, B=B, far=far, hot=hot,
                                 sinks=[0.0, 25.0, -3.0, 1.0], towers=[(119, 3), (101, 16)], tiles=True, scale=0.005, every=50)
    v = rows[:, 4 * 64 + 2 * 64:4 * 64 + 2 * 64 + Dv]
    for t in (dists[0], dists[-1], dists[-1] + 1, 64, 99, 100, 105, 119):
        keys = [t - d for d in dists if t - d >= 0]
        assert float((got[t, :Dv] - v[keys].mean(0)).abs().max()) < 0.06, t
    assert float(got[:, Dv:2 * Dv].abs().max()) < 1e-2          # head 1: swallowed by its sink, towers or not


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D", [(4, 1, 64), (8, 2, 128), (6, 6, 64)])
def test_split_kv_decode_kernel_takes_bias_and_sink(H, G, D):
    # the newest row of sequences of 1 .. 700 keys (one partition, several, a merge), as a decode batch
    dev, B, far, BS = "cuda:0", 14, 90, 16
    g = torch.Generator().manual_seed(H)
    lens = [1, 2, 17, 200, 700]
    relt = rounded(torch.randn(B, H, generator=g), torch.bfloat16)
    relt[9, 0] = 12.0                                   # distances 29 .. 37 tower for head 0
    sink = torch.tensor([0.0, 20.0, -30.0, 1.0, 0.5, -0.5, 2.0, 3.0][:H])
    C = H * D + 2 * G * D
    nb = sum(-(-n // BS) for n in lens)
    perm = np.random.default_rng(1).permutation(nb + 2)
    kc = torch.full((nb + 2, G, BS, D), 50.0, dtype=torch.bfloat16, device=dev)
    vc = torch.full((nb + 2, G, BS // 8, D, 8), 50.0, dtype=torch.bfloat16, device=dev)
    eye = torch.eye(C, dtype=F64)
    W = {"q": eye[:H * D], "k": eye[H * D:H * D + G * D], "v": eye[H * D + G * D:]}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "q_temp": {"coef": 0.3, "every": 64}}
    bt = np.zeros((len(lens), -(-max(lens) // BS)), dtype=np.int32)
    qs, want, used = [], [], 0
    for b, n in enumerate(lens):
        rows = rounded(torch.randn(n, C, generator=g) * 0.5, torch.bfloat16)
        k = -(-n // BS)
        bt[b, :k] = perm[used:used + k]
        used += k
        slots = [int(bt[b, t // BS]) * BS + t % BS for t in range(n)]
        q = ops.qk_norm_pages(rows.to(device=dev, dtype=torch.bfloat16), H, D, G, D, D, i32(np.arange(n), dev), i32(slots, dev),
                              1e-5, 0.3, 64, kc, vc)
        qs.append(q[-1])
        qw, kw_, vw = oracle.attention_qkv(W, "", m, rows.double(), 1e-5)
        want.append(oracle.attention_core(qw, kw_, vw, relt.double(), sink.double(), 0.05, far)[-1])
    out = ops.attn_decode(torch.stack(qs).view(len(lens), H, D), kc, vc, i32(bt, dev), i32(lens, dev), 0.05, max(lens),
                          dist_bias=ops.bucketed_bias(relt, far).to(dev), sink=sink.to(dev))
    assert rel(out.view(len(lens), -1), torch.stack(want)) < 3e-2
    assert float(out[:, 1].float().abs().max()) < 1e-2         # head 1: swallowed by its sink


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D", [(4, 1, 64), (4, 2, 128)])
def test_prefill_kernel_takes_bias_and_sink(H, G, D):
    # a batch of three portions: one continuing after 50 cached rows, one from position 0, one of a single row
    dev, B, far, BS = "cuda:0", 14, 90, 16
    g = torch.Generator().manual_seed(H + D)
    relt = rounded(torch.randn(B, H, generator=g), torch.bfloat16)
    relt[9, 0] = 12.0
    sink = torch.tensor([0.0, 20.0, -30.0, 1.0])
    C = H * D + 2 * G * D
    spans = [(50, 150), (0, 37), (20, 21)]              # (first row of the portion, end) per sequence
    nb = sum(-(-e // BS) for _, e in spans)
    perm = np.random.default_rng(2).permutation(nb + 2)
    kc = torch.full((nb + 2, G, BS, D), 50.0, dtype=torch.bfloat16, device=dev)
    vc = torch.full((nb + 2, G, BS // 8, D, 8), 50.0, dtype=torch.bfloat16, device=dev)
    eye = torch.eye(C, dtype=F64)
    W = {"q": eye[:H * D], "k": eye[H * D:H * D + G * D], "v": eye[H * D + G * D:]}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "q_temp": {"coef": 0.3, "every": 64}}
    bt = np.zeros((len(spans), -(-max(e for _, e in spans) // BS)), dtype=np.int32)
    qs, want, used = [], [], 0
    for b, (a, e) in enumerate(spans):
        rows = rounded(torch.randn(e, C, generator=g) * 0.5, torch.bfloat16)
        k = -(-e // BS)
        bt[b, :k] = perm[used:used + k]
        used += k
        slots = [int(bt[b, t // BS]) * BS + t % BS for t in range(e)]
        q = ops.qk_norm_pages(rows.to(device=dev, dtype=torch.bfloat16), H, D, G, D, D, i32(np.arange(e), dev), i32(slots, dev),
                              1e-5, 0.3, 64, kc, vc)
        qs.append(q[a:])
        qw, kw_, vw = oracle.attention_qkv(W, "", m, rows.double(), 1e-5)
        want.append(oracle.attention_core(qw, kw_, vw, relt.double(), sink.double(), 0.05, far)[a:])
    qlens = [e - a for a, e in spans]
    out = ops.attn_prefill(torch.cat(qs).view(-1, H, D), kc, vc, i32(np.cumsum([0] + qlens), dev), i32([e for _, e in spans], dev),
                           i32(bt, dev), 0.05, tiles=ops.prefill_tiles(qlens, dev),
                           dist_bias=ops.bucketed_bias(relt, far).to(dev), sink=sink.to(dev))
    assert rel(out.view(sum(qlens), -1), torch.cat(want)) < 3e-2
    assert float(out[:, 1].float().abs().max()) < 1e-2         # head 1: swallowed by its sink


# --------------------------------------------------------------------------------------- state-space mixer
def _mamba_weights(g, H, P, N, G, taps, keep_head0=False):
    C = H * P + 2 * G * N
    W = {"conv": torch.randn(C, taps, generator=g) * 0.5, "conv.b": torch.randn(C, generator=g) * 0.2,
         "dt_bias": torch.randn(H, generator=g), "A_log": torch.randn(H, generator=g) * 0.7, "D": torch.randn(H, generator=g),
         "norm": 1 + 0.2 * torch.randn(H * P, generator=g)}
    if keep_head0:
        W["A_log"][0] = -25.0          # exp(-exp(-25) dt) = 1 in fp32: head 0 forgets nothing
    return W


def _mamba_want(W, rows, H, P, N, G, taps, ng, eps):
    n = rows.shape[1]
    Wd = {k: v.double() for k, v in W.items()}
    Wd["in"], Wd["o"] = torch.eye(n, dtype=F64), torch.eye(H * P, dtype=F64)
    m = {"heads": H, "vdim": P, "state": N, "groups": G, "conv": taps, "norm_groups": ng}
    return oracle.mamba2(Wd, "", m, rows.double(), eps)


def _mamba_run(device, dtype, W, H, P, N, G, ng, eps, batch, tails, states):
    """batch: [(rows [n, width], first position, slot)] -> outputs per entry, one ops.mamba2 call."""
    Wf = {k: v.to(device) for k, v in W.items()}
    src = torch.cat([r for r, _, _ in batch]).to(device=device, dtype=dtype)
    cu = np.cumsum([0] + [r.shape[0] for r, _, _ in batch])
    pos = np.concatenate([np.arange(p0, p0 + r.shape[0]) for r, p0, _ in batch])
    out = ops.mamba2(src, H, P, N, G, Wf["conv"], Wf["conv.b"], Wf["dt_bias"], Wf["A_log"], Wf["D"], Wf["norm"], ng, eps,
                     i32(pos, device), i32(cu, device), i32([s for _, _, s in batch], device), tails, states,
                     max_rows=max(r.shape[0] for r, _, _ in batch))
    return [out[cu[k]:cu[k + 1]].float().cpu() for k in range(len(batch))]


@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("H,P,N,G,taps,ng", [(4, 8, 8, 2, 3, 2), (3, 7, 5, 3, 4, 3), (2, 10, 12, 1, 1, 1), (2, 64, 64, 2, 5, 4),
                                           (6, 4, 40, 2, 2, 1)])
def test_state_space_portions_state_slots_and_reuse(device, dtype, H, P, N, G, taps, ng):
    g = torch.Generator().manual_seed(H * P + N)
    width = 2 * H * P + 2 * G * N + H
    W = _mamba_weights(g, H, P, N, G, taps)
    eps = 1e-5
    a = rounded(torch.randn(41, width, generator=g), dtype)
    b = rounded(torch.randn(23, width, generator=g), dtype)
    wa, wb = _mamba_want(W, a, H, P, N, G, taps, ng, eps), _mamba_want(W, b, H, P, N, G, taps, ng, eps)
    tails, states = ops.mamba2_states(3, H, P, N, G, taps, dtype, device)
    tails.fill_(7.0)                                # leftovers of whoever held the slots before
    states.fill_(-3.0)
    t = tol(dtype) * 2.5
    # a in portions of 2, 9, 1, 1, 17, 11 in slot 2; b beside it from its third step on, in slot 0
    cuts_a, cuts_b = [2, 9, 1, 1, 17, 11], [None, None, 1, 2, 13, 7]
    ia = ib = 0
    for ca, cb in zip(cuts_a, cuts_b):
        batch = [(a[ia:ia + ca], ia, 2)]
        if cb:
            batch.insert(0, (b[ib:ib + cb], ib, 0))
        outs = _mamba_run(device, dtype, W, H, P, N, G, ng, eps, batch, tails, states)
        assert rel(outs[-1], wa[ia:ia + ca]) < t, ("a", ia)
        if cb:
            assert rel(outs[0], wb[ib:ib + cb]) < t, ("b", ib)
            ib += cb
        ia += ca
    # slot 2 is taken over by b from its start (zero state and zeros before the convolution, whatever a left), one row at a time
    got = torch.cat([_mamba_run(device, dtype, W, H, P, N, G, ng, eps, [(b[i:i + 1], i, 2)], tails, states)[0] for i in range(23)])
    assert rel(got, wb) < t


@pytest.mark.parametrize("device,dtype", MODES)
def test_state_space_head_that_forgets_nothing_over_a_long_run(device, dtype):
    # head 0 keeps everything: after 1100 rows its state still holds row 0's contribution in full.  Long portions
    # are scanned in segments on the GPU (the join multiplies each segment's decays), then 40 single rows
    H, P, N, G, taps, ng = 2, 8, 16, 1, 4, 1
    g = torch.Generator().manual_seed(11)
    width = 2 * H * P + 2 * G * N + H
    W = _mamba_weights(g, H, P, N, G, taps, keep_head0=True)
    n = 1140
    rows = rounded(torch.randn(n, width, generator=g) * 0.5, dtype)
    rows[:, -H:] -= 3.0                                  # small steps: the sum over a thousand rows stays moderate
    rows = rounded(rows, dtype)
    want = _mamba_want(W, rows, H, P, N, G, taps, ng, 1e-5)
    tails, states = ops.mamba2_states(2, H, P, N, G, taps, dtype, device)
    states.fill_(9.0)
    got = _mamba_run(device, dtype, W, H, P, N, G, ng, 1e-5, [(rows[:1100], 0, 1)], tails, states)
    got += [_mamba_run(device, dtype, W, H, P, N, G, ng, 1e-5, [(rows[i:i + 1], i, 1)], tails, states)[0] for i in range(1100, n)]
    assert rel(torch.cat(got), want) < tol(dtype) * 4
    # two long portions in one batch (segments of both), the second continuing from a state
    tails, states = ops.mamba2_states(2, H, P, N, G, taps, dtype, device)
    _mamba_run(device, dtype, W, H, P, N, G, ng, 1e-5, [(rows[:70], 0, 0)], tails, states)
    o = _mamba_run(device, dtype, W, H, P, N, G, ng, 1e-5, [(rows[70:700], 70, 0), (rows[:600], 0, 1)], tails, states)
    assert rel(o[0], want[70:700]) < tol(dtype) * 4 and rel(o[1], want[:600]) < tol(dtype) * 4


# --------------------------------------------------------------------------------------- router, experts
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("E,top,D", [(5, 2, 24), (12, 12, 37), (9, 1, 16), (70, 6, 40)])
def test_router_takes_the_largest_biased_logits_and_softmaxes_them(device, dtype, E, top, D):
    g = torch.Generator().manual_seed(E)
    x = rounded(torch.randn(6, D, generator=g), dtype)
    R, b = torch.randn(E, D, generator=g), torch.randn(E, generator=g) * 2
    b[E - 1] = 40.0                                     # the bias alone decides: the last expert is always chosen, first
    ids, wts = ops.router_softmax(x.to(device=device, dtype=dtype), R.to(device), b.to(device), top)
    W = {"router": R.double(), "router.b": b.double()}
    for t in range(6):
        chosen, _ = oracle.route(W, "", x[t].double(), top)
        assert [int(i) for i in ids[t]] == [e for e, _ in chosen]
        assert float((wts.view(6, top)[t].cpu().double() - torch.tensor([w for _, w in chosen])).abs().max()) < 1e-5
        assert int(ids[t, 0]) == E - 1


@pytest.mark.parametrize("device,dtype", MODES)
def test_clamped_pair_experts_beyond_both_limits(device, dtype):
    g = torch.Generator().manual_seed(3)
    T, D, F, E, top = 5, 24, 13, 4, 2
    x = rounded(torch.randn(T, D, generator=g), dtype)
    wg, wu = rounded(torch.randn(E, F, D, generator=g) * 0.8, dtype), rounded(torch.randn(E, F, D, generator=g) * 0.8, dtype)
    wd = rounded(torch.randn(E, D, F, generator=g) * 0.3, dtype)
    ids = torch.tensor([[0, 3], [1, 2], [3, 0], [2, 2], [1, 0]], dtype=torch.int32)
    wts = torch.rand(T * top, generator=g)
    y = ops.moe_pairs(x.to(device=device, dtype=dtype), wg.to(device=device, dtype=dtype), wu.to(device=device, dtype=dtype),
                      wd.to(device=device, dtype=dtype), ids.to(device), wts.to(device), clamp=(1.25, 1.702))
    want = torch.zeros(T, D, dtype=F64)
    for t in range(T):
        for k in range(top):
            e = int(ids[t, k])
            W = {"gate": wg[e].double(), "up": wu[e].double(), "down": wd[e].double()}
            want[t] += float(wts[t * top + k]) * oracle.expert(W, "", x[t:t + 1].double(), 1.25)[0]
    pre = x.double() @ wg[0].double().T
    assert float(pre.max()) > 1.25 and float((x.double() @ wu[0].double().T).min()) < -1.25     # the clamps bite
    assert rel(y, want) < tol(dtype) * 1.5
