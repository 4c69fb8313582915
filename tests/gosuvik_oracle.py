"""A plain, slow implementation of the Gosuvik design in float64: one function per mechanism, loops
over positions and heads, no cache, no batching, nothing shared with the package.

Notation: x_t the residual stream at position t (counted from 0 per sequence); W maps tensor names
to float tensors; cfg is the config.json dictionary; h the input of a sublayer.

  layer          x += mixer(N1 x);  x += ff(N2 x) (if any)
  N(y)           y cut into `groups` equal parts, each part / sqrt(mean(part^2) + eps), the whole times w
  loop           layers start .. stop - 1 run `times` times with the same weights; every pass is a run of its own
  channel_delta  q, k (G heads), v (H heads) <- silu(conv(W h));  q, k <- unit length (1e-6 inside the root), q *= dk^-1/2
                 beta = sigmoid(Wb h);  g = exp(-exp(A_log[head]) softplus(Wa2 Wa1 h + dt_bias))  (one decay per key channel)
                 S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
                 out = Wo [o / rms(o) * w * sigmoid(Wg2 Wg1 h)]
  latent         [c | kr] = Wdkv h;  c <- c / rms(c) * w;  k_head = [Wuk c | rot(kr)];  v_head = Wuv c;  q_head = [qn | rot(qr)]
                 softmax over the last `window` positions;  out = Wo [heads * sigmoid(Wg h)]
  left           q, k <- per-head RMS norm with a weight, then rotation;  v_j rotated by j over its whole width;
                 p_ij = exp(s_ij) / (sum_j exp(s_ij) + exp(sink_head)) over the last `window` positions;
                 head output rotated back by -i;  Wo
  right          i~ = cap tanh((Wi h + bi) / cap);  f~ = logsigmoid(cap tanh((Wf h + bf) / cap));  m' = max(f~ + m, i~)
                 S <- exp(f~ + m - m') S + exp(i~ - m') k v^T;  n likewise with k;  o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)
                 out = Wo [o / rms(o) per head * w * sigmoid(Wg h)]
  parallel       left_scale * left + right_scale * right
  dense ff       z = Wup h;  Wdown (a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e)
  experts        Wdown (silu(Wgate h) * Wup h), the `top` largest of softmax(Wr h), weights divided by their sum
  output         N_final(x), head
"""
import math

import torch

F64 = torch.float64


def unit_rms(y, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def group_norm(y, w, eps, groups):
    T, D = y.shape
    return (unit_rms(y.reshape(T, groups, D // groups), eps)).reshape(T, D) * w


def silu(z):
    return z / (1.0 + torch.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_conv(x, w):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, taps - 1 - j] x_(t - j), nothing before position 0."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            if t - j >= 0:
                y[t] += w[:, taps - 1 - j] * x[t - j]
    return y


# ------------------------------------------------------------------------------------------ rotation
def rot_table(dims, base, scaling=None):
    """(frequencies [dims / 2], magnitude of cos / sin)."""
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    mag = 1.0
    if scaling and "original" in scaling:
        factor = scaling["factor"]
        d_of = lambda turns: dims * math.log(scaling["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))  # noqa: E731
        lo = max(math.floor(d_of(scaling["fast"])), 0)
        hi = min(math.ceil(d_of(scaling["slow"])), dims - 1)
        for i in range(half):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    elif scaling:
        f = [x / scaling["factor"] for x in f]
    return f, mag


def rotate_halves(vec, p, freqs, mag=1.0, off=0):
    """vec [..., d]: dims off + i and off + i + len(freqs) turned by the angle p * freqs[i]."""
    out = vec.clone()
    half = len(freqs)
    for i, f in enumerate(freqs):
        a = p * f
        c, s = math.cos(a) * mag, math.sin(a) * mag
        u, v = vec[..., off + i], vec[..., off + i + half]
        out[..., off + i] = u * c - v * s
        out[..., off + i + half] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------ mixers
def channel_delta(W, p, m, h, eps):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(T, G, dk)
    k = silu(causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(T, G, dk)
    v = silu(causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(h @ W[p + "b"].T)                                              # [T, H]
    dt = softplus((h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]).view(T, H, dk)
    g = torch.exp(-torch.exp(W[p + "A_log"]).view(1, H, 1) * dt)
    gate = sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        grp = hd // (H // G)
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = g[t, hd].unsqueeze(1) * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, grp])
            S = S + torch.outer(k[t, grp], u)
            o[t, hd] = S.T @ q[t, grp]
    o = unit_rms(o, eps) * W[p + "norm"] * gate
    return o.reshape(T, H * dv) @ W[p + "o"].T


def latent_attention(W, p, m, h, eps):
    T = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    freqs, mag = rot_table(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    window = (m.get("mask") or {}).get("size") or 0
    q = (h @ W[p + "q"].T).view(T, H, dn + dr)
    ckr = h @ W[p + "dkv"].T
    c = unit_rms(ckr[:, :r], eps) * W[p + "dkv.norm"]
    kr = ckr[:, r:]
    kn = (c @ W[p + "uk"].T).view(T, H, dn)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    for t in range(T):
        q[t] = rotate_halves(q[t], t, freqs, mag, off=dn)
        kr[t] = rotate_halves(kr[t], t, freqs, mag)
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        lo = max(0, t - window + 1) if window else 0
        for hd in range(H):
            s = (kn[lo:t + 1, hd] @ q[t, hd, :dn] + kr[lo:t + 1] @ q[t, hd, dn:]) * m["scale"]
            pr = torch.softmax(s, 0)
            out[t, hd] = pr @ v[lo:t + 1, hd]
    out = out.reshape(T, H * dv) * sigmoid(h @ W[p + "g"].T)
    return out @ W[p + "o"].T


def sink_attention(W, p, m, h, eps):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    freqs, mag = rot_table(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    vfreqs, _ = rot_table(dv, m["rot"]["base"])
    window = (m.get("mask") or {}).get("size") or 0
    q = unit_rms((h @ W[p + "q"].T).view(T, H, dk), eps) * W[p + "q.norm"]
    k = unit_rms((h @ W[p + "k"].T).view(T, G, dk), eps) * W[p + "k.norm"]
    v = (h @ W[p + "v"].T).view(T, G, dv)
    for t in range(T):
        q[t] = rotate_halves(q[t], t, freqs, mag)
        k[t] = rotate_halves(k[t], t, freqs, mag)
        v[t] = rotate_halves(v[t], t, vfreqs)
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        lo = max(0, t - window + 1) if window else 0
        for hd in range(H):
            grp = hd // (H // G)
            s = (k[lo:t + 1, grp] @ q[t, hd]) * m["scale"]
            mx = max(float(s.max()), float(W[p + "sink"][hd]))
            e = torch.exp(s - mx)
            pr = e / (e.sum() + math.exp(float(W[p + "sink"][hd]) - mx))
            out[t, hd] = rotate_halves(pr @ v[lo:t + 1, grp], -t, vfreqs)
    return out.reshape(T, H * dv) @ W[p + "o"].T


def matrix_memory(W, p, m, h, eps):
    T = h.shape[0]
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ W[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, dk)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    ig = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    o = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        n = torch.zeros(dk, dtype=F64)
        mx = 0.0
        for t in range(T):
            i_t, f_t = float(ig[t, hd]), float(fg[t, hd])
            m_new = max(f_t + mx, i_t)
            a, b = math.exp(f_t + mx - m_new), math.exp(i_t - m_new)
            S = a * S + b * torch.outer(k[t, hd], v[t, hd])
            n = a * n + b * k[t, hd]
            mx = m_new
            o[t, hd] = (S.T @ q[t, hd]) / (max(abs(float(n @ q[t, hd])), math.exp(-mx)) + 1e-6)
    o = unit_rms(o, eps).reshape(T, H * dv) * W[p + "norm"] * sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def parallel(W, p, m, h, eps):
    return (m["left_scale"] * sink_attention(W, p + "left.", m["left"], h, eps)
            + m["right_scale"] * matrix_memory(W, p + "right.", m["right"], h, eps))


MIXERS = {"channel_delta": channel_delta, "latent_attention": latent_attention, "parallel": parallel}


# ------------------------------------------------------------------------------------------ feed-forwards
def poly_ff(W, p, h, eps):
    z = h @ W[p + "up"].T
    a, b, c, e = (float(x) for x in W[p + "act"])
    y = a * unit_rms(z, eps) + b * unit_rms(z ** 2, eps) + c * unit_rms(z ** 3, eps) + e
    return y @ W[p + "down"].T


def router(W, p, f, h):
    """(chosen experts [T, top], their weights [T, top], margin [T]: the last chosen logit minus the first one
    left out, in units of the logits' spread; infinite when every expert is chosen)."""
    z = h @ W[p + "router"].T
    s = torch.softmax(z, -1)
    top = f["router"]["top"]
    val, idx = torch.sort(s, dim=-1, descending=True, stable=True)
    w = val[:, :top] / (val[:, :top].sum(-1, keepdim=True) + 1e-20)
    if top < s.shape[1]:
        zs = torch.sort(z, dim=-1, descending=True).values
        margin = (zs[:, top - 1] - zs[:, top]) / z.std(-1).clamp_min(1e-9)
    else:
        margin = torch.full((h.shape[0],), float("inf"), dtype=F64)
    return idx[:, :top], w, margin


def expert_ff(W, p, f, h, margins=None):
    ids, w, margin = router(W, p, f, h)
    if margins is not None:
        for t in range(h.shape[0]):
            margins[t] = min(margins[t], float(margin[t]))
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e, we in zip(ids[t].tolist(), w[t]):
            q = p + f"e{e}."
            out[t] += we * ((silu(h[t] @ W[q + "gate"].T) * (h[t] @ W[q + "up"].T)) @ W[q + "down"].T)
    return out


# ------------------------------------------------------------------------------------------ the model
def runs(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, times = lp["start"], lp["stop"], lp["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg, W, tokens, streams=None, margins=None):
    """float64 logits [T, vocab] of one sequence; streams (a list) receives x after every layer run;
    margins (a list of T floats) is lowered to every position's smallest router margin."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i in runs(cfg):
        L = cfg["layers"][i]
        p = f"l{i}."
        x = x + MIXERS[L["type"]](W, p + "mix.", L["mixer"], group_norm(x, W[p + "norm1"], eps, groups), eps)
        f = L.get("mlp")
        if f:
            hn = group_norm(x, W[p + "norm2"], eps, groups)
            x = x + (poly_ff(W, p + "mlp.", hn, eps) if f["kind"] == "dense" else expert_ff(W, p + "mlp.", f, hn, margins))
        if streams is not None:
            streams.append(x.clone())
    return group_norm(x, W["final.norm"], eps, groups) @ W["head"].T
