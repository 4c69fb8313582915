"""A plain, slow implementation of the Vinozen design in float64: one function per mechanism, loops
over positions and heads, no cache, no batching, nothing shared with the package.

Notation: x_t the residual stream at position t (counted from 0 per sequence); W maps tensor names
to float tensors; cfg is the config.json dictionary.

  embedding    x_t = E[tok_t] * s + pe(t),  pe(t)[2i] = sin(t w_i), pe(t)[2i + 1] = cos(t w_i), w_i = 10000^(-2i / D)
  layer        x += LN1(mixer(x));  x += LN2(ff(x)) (if any);  x += side(x, tok)
  LN(y)        (y - mean y) / sqrt(var y + eps) * w   (var = mean squared deviation)
  side         e = E_side[tok, i d:(i + 1) d];  g = gelu_tanh(Wg x) * e;  y = Wp g;  y / sqrt(mean y^2 + eps) * w
  attention    q, k unit-RMS per head;  q *= 1 + c ln(floor((t + 1) / every) + 1);
               s_tj = scale q_t . k_j + rel[bucket(t - j), head];  p = exp(s) / (sum_j exp(s) + exp(sink))
  mamba2       [z | x | B | C | dt] = W_in h;  [x | B | C] = silu(conv(.) + b);  dt = softplus(dt + dt_bias)
               S = exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D x;  y = groupRMS(y silu(z)) * w
  experts      g = min(Wg h, L), u = clamp(Wu h, -L, L);  Wd (g sigmoid(1.702 g) (u + 1))
  router       z = Wr h + b;  the `top` largest;  weights softmax over those
  output       LN_final(x) . E^T
"""
import math

import torch

F64 = torch.float64


def layer_norm(y, w, eps):
    mu = y.mean(-1, keepdim=True)
    var = ((y - mu) ** 2).mean(-1, keepdim=True)
    return (y - mu) / torch.sqrt(var + eps) * w


def unit_rms(y, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def sinusoid(t, D):
    pe = torch.zeros(D, dtype=F64)
    for c in range(D):
        ang = t * 10000.0 ** (-2.0 * (c // 2) / D)
        pe[c] = math.sin(ang) if c % 2 == 0 else math.cos(ang)
    return pe


def bucket(n, B, far):
    """Bucket of distance n >= 0 among B: the first B // 2 distances exactly, the rest logarithmically up to `far`."""
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (B - half))))


def temperature(t, coef, every):
    return 1.0 + coef * math.log((t + 1) // every + 1) if every else 1.0


def attention_qkv(W, p, m, h, eps, with_kv=True):
    """(q [T, H, dk] normed and tempered, k [T, G, dk] normed, v [T, G, dv]) of one layer's own projections."""
    T, H, G, dk, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    qt = m.get("q_temp") or {}
    q = unit_rms((h @ W[p + "q"].T).view(T, H, dk), eps)
    for t in range(T):
        q[t] = q[t] * temperature(t, qt.get("coef", 0.0), qt.get("every", 0))
    if not with_kv:
        return q, None, None
    return q, unit_rms((h @ W[p + "k"].T).view(T, G, dk), eps), (h @ W[p + "v"].T).view(T, G, dv)


def attention_core(q, k, v, rel, sink, scale, far):
    """Per-position loop: head h attends over keys 0..t of its group with the bucketed bias and the sink."""
    T, H, _ = q.shape
    G, B = k.shape[1], rel.shape[0]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for t in range(T):
        for hd in range(H):
            g = hd // (H // G)
            s = torch.stack([scale * (q[t, hd] @ k[j, g]) + rel[bucket(t - j, B, far), hd] for j in range(t + 1)])
            mx = max(float(s.max()), float(sink[hd]))
            e = torch.exp(s - mx)
            den = e.sum() + math.exp(float(sink[hd]) - mx)
            out[t, hd] = (e / den) @ v[:t + 1, g]
    return out.reshape(T, -1)


def mamba2(W, p, m, h, eps):
    T, H, P, N, G, taps = h.shape[0], m["heads"], m["vdim"], m["state"], m.get("groups", 1), m["conv"]
    ng = m.get("norm_groups", 1)
    inner = H * P
    u = h @ W[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    cw, cb = W[p + "conv"], W[p + "conv.b"]
    conv = torch.zeros_like(xbc)
    for t in range(T):
        acc = cb.clone()
        for j in range(taps):                      # last column: the current token
            src = t - (taps - 1) + j
            if src >= 0:
                acc = acc + cw[:, j] * xbc[src]
        conv[t] = silu(acc)
    xs, Bm, Cm = conv[:, :inner].view(T, H, P), conv[:, inner:inner + G * N].view(T, G, N), conv[:, inner + G * N:].view(T, G, N)
    dt = torch.log1p(torch.exp(dt + W[p + "dt_bias"]))
    y = torch.zeros(T, H, P, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        a = -math.exp(float(W[p + "A_log"][hd]))
        for t in range(T):
            S = math.exp(a * float(dt[t, hd])) * S + dt[t, hd] * torch.outer(Bm[t, g], xs[t, hd])
            y[t, hd] = S.T @ Cm[t, g] + W[p + "D"][hd] * xs[t, hd]
    y = y.reshape(T, inner) * silu(z)
    y = unit_rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def dense_ff(W, p, h):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def expert(W, p, h, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def route(W, p, h, top):
    """([(expert, weight)], margin) of one row: the `top` largest logits, softmax over them; margin: how far
    the last chosen logit lies above the first one left out, in units of the logits' spread."""
    z = W[p + "router"] @ h + (W[p + "router.b"] if p + "router.b" in W else 0.0)
    ranked = sorted(range(z.shape[0]), key=lambda e: (-float(z[e]), e))
    order = ranked[:top]
    mx = max(float(z[e]) for e in order)
    ex = [math.exp(float(z[e]) - mx) for e in order]
    margin = math.inf if top >= len(ranked) else float(z[ranked[top - 1]] - z[ranked[top]]) / max(float(z.std()), 1e-9)
    return [(e, x / sum(ex)) for e, x in zip(order, ex)], margin


def moe_ff(W, p, f, h, margins=None):
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen, margin = route(W, p, h[t], f["router"]["top"])
        if margins is not None:
            margins[t] = min(margins[t], margin)
        for e, w in chosen:
            out[t] += w * expert(W, p + f"e{e}.", h[t:t + 1], f["expert"]["limit"])[0]
    if f.get("shared"):
        out = out + expert(W, p + "shared.", h, f["shared"]["limit"])
    return out


def side_input(W, p, x, side_rows, eps):
    y = (gelu_tanh(x @ W[p + "gate"].T) * side_rows) @ W[p + "proj"].T
    return unit_rms(y, eps) * W[p + "norm"]


def forward(tokens, W, cfg, layers_out=None, margins=None):
    """float64 logits [T, vocab] of one sequence; layers_out receives the stream after every layer;
    margins (a list of T floats, +inf) the smallest router margin of every position over the layers."""
    W = {k: v.to(F64) for k, v in W.items()}
    T, D, eps = len(tokens), cfg["width"], cfg["norm"]["eps"]
    tok = torch.tensor(tokens, dtype=torch.long)
    x = W["embed"][tok] * (cfg.get("embedding") or {}).get("scale", 1.0)
    x = x + torch.stack([sinusoid(t, D) for t in range(T)])
    sd = (cfg.get("token_side") or {}).get("dim", 0)
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        if L["type"] == "attention":
            own = m.get("kv_from") is None
            q, k, v = attention_qkv(W, p + "mix.", m, x, eps, with_kv=own)
            if own:
                kv[i] = (k, v)
            k, v = kv[i if own else m["kv_from"]]
            a = attention_core(q, k, v, W[p + "mix.rel"], W[p + "mix.sink"], m["scale"], m["bias_max"]) @ W[p + "mix.o"].T
        else:
            a = mamba2(W, p + "mix.", m, x, eps)
        x = x + layer_norm(a, W[p + "norm1"], eps)
        f = L.get("mlp")
        if f:
            y = dense_ff(W, p + "mlp.", x) if f["kind"] == "dense" else moe_ff(W, p + "mlp.", f, x, margins)
            x = x + layer_norm(y, W[p + "norm2"], eps)
        if sd:
            x = x + side_input(W, p + "side.", x, W["side.embed"][tok][:, i * sd:(i + 1) * sd], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return layer_norm(x, W["final.norm"], eps) @ W["embed"].T
