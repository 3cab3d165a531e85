"""Plain float64 implementation of the Pironex design, one function per
mechanism, written token by token from the equations. It shares no code with
the product path; the tests compare the engine with it.

A model is (cfg, w): cfg is the checkpoint's config.json as a dict, w maps
checkpoint tensor names to float64 tensors.

    x0 = embed[t] * s
    layer i:   u = x + ln(mixer(canon1(ln(x) w1))) w1b
               X_{i+1} = u + ln(ff(canon2(ln(u) w2))) w2b        (no ff: X_{i+1} = u)
               x <- sum_{j <= i+1} dwa_i[j] X_j                  (X_0 = x0)
    logits = embed . (ln(x) w_final)

ln = (v - mean) / sqrt(var + eps), canon(h)_t = h_t + sum_j c[:, j] h_{t-K+1+j}.
"""

import math

import torch

F64 = torch.float64


# --- small pieces -----------------------------------------------------------------

def layer_norm(v, w, eps):
    mu = v.mean(-1, keepdim=True)
    var = ((v - mu) ** 2).mean(-1, keepdim=True)
    return (v - mu) / torch.sqrt(var + eps) * w


def rms(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def canon(h, c):
    """h [T, W], c [W, K]: h_t + sum_j c[:, j] h_{t-K+1+j}, zeros before the start."""
    T, _ = h.shape
    K = c.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                out[t] += c[:, j] * h[s]
    return out


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate(vec, p, base, dims, layout):
    """Rotary position on the first ``dims`` entries of vec [..., D] at position p.
    layout 'half': entry i pairs with i + dims/2; 'pairs': 2i with 2i+1."""
    out = vec.clone()
    for i in range(dims // 2):
        a = p * base ** (-2.0 * i / dims)
        i0, i1 = (i, i + dims // 2) if layout == "half" else (2 * i, 2 * i + 1)
        u, v = vec[..., i0], vec[..., i1]
        out[..., i0] = u * math.cos(a) - v * math.sin(a)
        out[..., i1] = v * math.cos(a) + u * math.sin(a)
    return out


def softmax_mix(scores, values):
    """scores: list of floats, values: list of vectors."""
    s = torch.stack(scores)
    p = torch.softmax(s, 0)
    return (p[:, None] * torch.stack(values)).sum(0)


# --- attention with a sliding window and pooled blocks --------------------------------

def visible(i, size, pool):
    """(token positions, pooled block numbers) that position i sees."""
    if not size:
        return list(range(i + 1)), []
    toks = [j for j in range(i + 1) if i - j < size]
    blocks = []
    if pool:
        b = 0
        while b * pool + pool - 1 <= i - size:
            blocks.append(b)
            b += 1
    return toks, blocks


def window_pool_attention(q, k, v, scale, softcap, size, pool):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] as the cache holds them (normed,
    rotated). Returns [T, H, Dv]."""
    T, H, D = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for i in range(T):
        toks, blocks = visible(i, size, pool)
        for h in range(H):
            g = h // rep
            keys = [k[b * pool:(b + 1) * pool, g].mean(0) for b in blocks] + [k[j, g] for j in toks]
            vals = [v[b * pool:(b + 1) * pool, g].mean(0) for b in blocks] + [v[j, g] for j in toks]
            sc = []
            for kk in keys:
                s = (q[i, h] * kk).sum() * scale
                if softcap:
                    s = softcap * torch.tanh(s / softcap)
                sc.append(s)
            out[i, h] = softmax_mix(sc, vals)
    return out


def attention_keys(w, pre, m, h, eps):
    """The cached keys and values of an attention layer with projections of
    its own: whole-projection RMS norm on k, then the rotation. h [T, W]."""
    T = h.shape[0]
    G, D, Dv = m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    k = rms(h @ w[pre + "k"].T, eps) * w[pre + "k.norm"]
    k = k.view(T, G, D)
    if rot.get("dims"):
        k = torch.stack([rotate(k[t], t, rot["base"], rot["dims"], "half") for t in range(T)])
    v = (h @ w[pre + "v"].T).view(T, G, Dv)
    return k, v


def attention_mixer(w, pre, m, h, eps, kv):
    """kv: (k, v) of the layer this one takes its keys and values from."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    rot = m.get("rot") or {}
    q = rms(h @ w[pre + "q"].T, eps) * w[pre + "q.norm"]
    q = q.view(T, H, D)
    if rot.get("dims"):
        q = torch.stack([rotate(q[t], t, rot["base"], rot["dims"], "half") for t in range(T)])
    mask = m.get("mask") or {}
    o = window_pool_attention(q, kv[0], kv[1], m["scale"], m.get("softcap") or 0.0, mask.get("size") or 0,
                              mask.get("pool") or 0)
    return o.reshape(T, -1) @ w[pre + "o"].T


# --- mamba2 ---------------------------------------------------------------------------

def silu(z):
    return z * torch.sigmoid(z)


def mamba2_mixer(w, pre, m, h, eps):
    T = h.shape[0]
    H, P, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * P
    y = h @ w[pre + "in"].T
    z, xbc, dt = y[:, :inner], y[:, inner:2 * inner + 2 * G * N], y[:, 2 * inner + 2 * G * N:]
    cw, cb = w[pre + "conv"], w[pre + "conv.b"]
    conv = torch.zeros_like(xbc)
    for t in range(T):
        acc = cb.clone()
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                acc = acc + cw[:, j] * xbc[s]
        conv[t] = silu(acc)
    x = conv[:, :inner].view(T, H, P)
    B = conv[:, inner:inner + G * N].view(T, G, N)
    C = conv[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + w[pre + "dt_bias"])
    A = torch.exp(w[pre + "A_log"])
    S = torch.zeros(H, N, P, dtype=F64)
    out = torch.zeros(T, H, P, dtype=F64)
    for t in range(T):
        for hd in range(H):
            g = hd // (H // G)
            S[hd] = math.exp(-float(A[hd]) * float(dt[t, hd])) * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            out[t, hd] = S[hd].T @ C[t, g] + w[pre + "D"][hd] * x[t, hd]
    gated = out.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    normed = rms(gated.view(T, ng, inner // ng), eps).reshape(T, inner) * w[pre + "norm"]
    return normed @ w[pre + "o"].T


# --- latent attention -------------------------------------------------------------------

def latent_mixer(w, pre, m, h, eps):
    T = h.shape[0]
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base = m["rot"]["base"]
    size = (m.get("mask") or {}).get("size") or 0
    q = (h @ w[pre + "q"].T).view(T, H, D + R)
    d = h @ w[pre + "dkv"].T
    c = rms(d[:, :C], eps) * w[pre + "dkv.norm"]
    kr = torch.stack([rotate(d[t, C:], t, base, R, "pairs") for t in range(T)])
    kn = (c @ w[pre + "uk"].T).view(T, H, D)
    vv = (c @ w[pre + "uv"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=F64)
    for i in range(T):
        toks, _ = visible(i, size, 0)
        for hd in range(H):
            qr = rotate(q[i, hd, D:], i, base, R, "pairs")
            sc = [((q[i, hd, :D] * kn[j, hd]).sum() + (qr * kr[j]).sum()) * m["scale"] for j in toks]
            out[i, hd] = softmax_mix(sc, [vv[j, hd] for j in toks])
    return out.reshape(T, -1) @ w[pre + "o"].T


# --- feed-forward -----------------------------------------------------------------------

def expert(w, pre, h, limit):
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def route(z, top):
    """(chosen experts, weights) of one token; ties go to the lower index."""
    order = sorted(range(len(z)), key=lambda e: (-float(z[e]), e))[:top]
    wts = torch.softmax(torch.stack([z[e] for e in order]), 0)
    return order, wts


def moe(w, pre, mlp, h):
    T = h.shape[0]
    out = torch.zeros_like(h)
    r = mlp["router"]
    for t in range(T):
        z = w[pre + "router"] @ h[t]
        order, wts = route(z, r["top"])
        for e, wt in zip(order, wts):
            out[t] += wt * expert(w, f"{pre}e{e}.", h[t], mlp["expert"]["limit"])
        sh = mlp.get("shared")
        if sh:
            gate = torch.sigmoid((w[pre + "shared.sg"] @ h[t])[0])
            out[t] += gate * expert(w, pre + "shared.", h[t], sh["limit"])
    return out


# --- the model ----------------------------------------------------------------------------

def forward(cfg, w, tokens, want_layers=False):
    """Logits [T, vocab] of one sequence (float64); with want_layers also the
    stream after every layer (after the depth average)."""
    eps = cfg["norm"]["eps"]
    ids = torch.tensor(tokens, dtype=torch.long)
    x = w["embed"][ids] * cfg["embedding"]["scale"]
    streams = [x]
    kvs = {}
    after = []
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}."
        m = L["mixer"]
        h = canon(layer_norm(x, w[pre + "norm1"], eps), w[pre + "canon1"])
        if L["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = attention_keys(w, pre + "mix.", m, h, eps)
                src = i
            a = attention_mixer(w, pre + "mix.", m, h, eps, kvs[src])
        elif L["type"] == "mamba2":
            a = mamba2_mixer(w, pre + "mix.", m, h, eps)
        elif L["type"] == "latent_attention":
            a = latent_mixer(w, pre + "mix.", m, h, eps)
        else:
            raise ValueError(L["type"])
        x = x + layer_norm(a, w[pre + "norm1b"], eps)
        if L.get("mlp"):
            h = canon(layer_norm(x, w[pre + "norm2"], eps), w[pre + "canon2"])
            x = x + layer_norm(moe(w, pre + "mlp.", L["mlp"], h), w[pre + "norm2b"], eps)
        streams.append(x)
        x = sum(w[pre + "dwa"][j] * streams[j] for j in range(i + 2))
        after.append(x)
    logits = layer_norm(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, after) if want_layers else logits


# --- random checkpoints ---------------------------------------------------------------------

def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    K = cfg["canon"]["taps"]
    s = {"embed": (V, W), "final.norm": (W,)}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = L["mixer"]
        s[p + "norm1"] = s[p + "norm1b"] = (W,)
        s[p + "canon1"] = (W, K)
        s[p + "dwa"] = (i + 2,)
        if L["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            s[p + "mix.q"], s[p + "mix.q.norm"] = (H * D, W), (H * D,)
            if m.get("kv_from") is None:
                s[p + "mix.k"], s[p + "mix.k.norm"], s[p + "mix.v"] = (G * D, W), (G * D,), (G * Dv, W)
            s[p + "mix.o"] = (W, H * Dv)
        elif L["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = H * P, H * P + 2 * G * N
            s[p + "mix.in"] = (inner + ch + H, W)
            s[p + "mix.conv"], s[p + "mix.conv.b"] = (ch, m["conv"]), (ch,)
            s[p + "mix.dt_bias"] = s[p + "mix.A_log"] = s[p + "mix.D"] = (H,)
            s[p + "mix.norm"], s[p + "mix.o"] = (inner,), (W, inner)
        else:
            H, D, R, Vd, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            s[p + "mix.q"], s[p + "mix.dkv"], s[p + "mix.dkv.norm"] = (H * (D + R), W), (C + R, W), (C,)
            s[p + "mix.uk"], s[p + "mix.uv"], s[p + "mix.o"] = (H * D, C), (H * Vd, C), (W, H * Vd)
        mlp = L.get("mlp")
        if mlp:
            s[p + "norm2"] = s[p + "norm2b"] = (W,)
            s[p + "canon2"] = (W, K)
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                s[f"{p}mlp.e{e}.gate"] = s[f"{p}mlp.e{e}.up"] = (ff, W)
                s[f"{p}mlp.e{e}.down"] = (W, ff)
            s[p + "mlp.router"] = (mlp["router"]["experts"], W)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                s[p + "mlp.shared.gate"] = s[p + "mlp.shared.up"] = (sf, W)
                s[p + "mlp.shared.down"], s[p + "mlp.shared.sg"] = (W, sf), (1, W)
    return s


def random_weights(cfg, seed=0):
    """Random tensors under the checkpoint's names, rounded to bfloat16 (as a
    checkpoint stores them) and returned in float64."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if name.endswith("q.norm") or name.endswith("k.norm") or leaf in ("norm", "norm1", "norm2", "norm1b", "norm2b"):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf in ("canon1", "canon2"):
            t = 0.4 * torch.randn(shape, generator=g)
        elif leaf == "dwa":
            t = 0.2 * torch.randn(shape, generator=g)
            t[-1] += 1.0
        elif leaf == "conv":
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf in ("b", "dt_bias", "D"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf == "A_log":
            t = torch.randn(shape, generator=g) - 1.0
        elif leaf == "embed":
            t = torch.randn(shape, generator=g)
        elif leaf == "router":
            t = 2.0 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        w[name] = t.bfloat16().to(F64)
    return w
