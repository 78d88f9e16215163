"""Plain, slow restatement of the layer-described Pamulix design in float64 numpy: one function per mechanism, the whole sequence at once, no cache.
It shares no code with the serving store; the tests compare the store's residual streams and logits with it.

Notation: x [T, width] residual stream; pos [T] positions from 0; W matrices are [out, in] and applied as x @ W.T; a layer is
x <- x + m * LN1(mixer(x)), then x <- x + m * LN2(ff(x)): the sublayers read x itself, the norm sits on their OUTPUT."""
import json
import math
import struct

import numpy as np


def bf16_round(a):
    """float32 array -> the nearest bfloat16 values (round to nearest even), returned as float32"""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def to_bf16_bits(a):
    return (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)


# ---------------------------------------------------------------------------------------------------------------- norms
def centered_norm(y, w, eps):
    """layer norm with a weight and no bias"""
    mu = y.mean(-1, keepdims=True)
    var = ((y - mu) ** 2).mean(-1, keepdims=True)
    return (y - mu) / np.sqrt(var + eps) * w


def rms_norm(y, w, eps):
    return y / np.sqrt((y ** 2).mean(-1, keepdims=True) + eps) * w


# ---------------------------------------------------------------------------------------------------------------- rotation
def yarn_table(dims, base, factor, original, fast, slow):
    """frequencies [dims / 2] and the factor on cos and sin: pairs that turn fast keep their frequency, slow ones are divided by `factor`, with a
    linear ramp between the pair indices at which `fast` and `slow` whole turns fit into `original` positions"""
    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_of(fast)), 0)
    hi = min(math.ceil(pair_of(slow)), dims - 1)
    f = np.zeros(dims // 2)
    for i in range(dims // 2):
        fi = base ** (-2.0 * i / dims)
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        f[i] = fi / factor * ramp + fi * (1.0 - ramp)
    return f, 0.1 * math.log(factor) + 1.0


def plain_table(dims, base):
    return np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)]), 1.0


def rotate_pairs(x, pos, freqs, mult):
    """x [T, heads, n]: coordinates (2i, 2i + 1), i < len(freqs), turn by pos * freqs[i]; cos and sin carry `mult`; the rest stays"""
    y = x.copy()
    for i, f in enumerate(freqs):
        ang = pos.astype(np.float64) * f
        c, s = (np.cos(ang) * mult)[:, None], (np.sin(ang) * mult)[:, None]
        a, b = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        y[:, :, 2 * i] = a * c - b * s
        y[:, :, 2 * i + 1] = b * c + a * s
    return y


def rot_table(rot):
    sc = rot.get("scaling")
    if sc:
        return yarn_table(rot["dims"], rot["base"], sc["factor"], sc["original"], sc["fast"], sc["slow"])
    return plain_table(rot["dims"], rot["base"])


# ---------------------------------------------------------------------------------------------------------------- attention with keys through a latent
def causal_softmax_attention(q, k, v, scale):
    """q [T, H, d], k [T, H, d], v [T, H, dv]: every j <= i, ordinary softmax"""
    T, H, _ = q.shape
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        for i in range(T):
            sc = (k[:i + 1, h] @ q[i, h]) * scale
            e = np.exp(sc - sc.max())
            out[i, h] = (e / e.sum()) @ v[:i + 1, h]
    return out


def latent_attention(h, W, p, m, pos, eps):
    """queries through a normed latent; keys and values of every head are expanded from ONE normed latent per token; a rotated key part is shared by
    the heads.  A head's query / key is [dim plain | rot_dim rotated]."""
    T = h.shape[0]
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    freqs, mult = rot_table(m["rot"])
    cq = rms_norm(h @ W[p + ".dq"].T, W[p + ".dq.norm"], eps)
    q = (cq @ W[p + ".uq"].T).reshape(T, H, d + r)
    q = np.concatenate([q[:, :, :d], rotate_pairs(q[:, :, d:], pos, freqs, mult)], -1)
    ckv = h @ W[p + ".dkv"].T
    c = rms_norm(ckv[:, :R], W[p + ".dkv.norm"], eps)
    kr = rotate_pairs(ckv[:, None, R:], pos, freqs, mult)                   # [T, 1, r]
    k = np.concatenate([(c @ W[p + ".uk"].T).reshape(T, H, d), np.repeat(kr, H, 1)], -1)
    v = (c @ W[p + ".uv"].T).reshape(T, H, dv)
    a = causal_softmax_attention(q, k, v, m["scale"])
    return a.reshape(T, H * dv) @ W[p + ".o"].T


# ---------------------------------------------------------------------------------------------------------------- chunked attention with a distance bias
def head_slopes(H):
    return np.array([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])


def chunked_bias_attention(q, k, v, scale, chunk):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query i sees j <= i of its own chunk of `chunk` positions (chunk 0: all j <= i); the score loses
    slope_h * (i - j); weights = exp(s_j) / (1 + sum exp(s_j)): a sink of score 0 without a value"""
    T, H, _ = q.shape
    G = k.shape[1]
    slopes = head_slopes(H)
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = (i // chunk) * chunk if chunk > 0 else 0
            sc = (k[lo:i + 1, g] @ q[i, h]) * scale - slopes[h] * (i - np.arange(lo, i + 1))
            mx = max(sc.max(), 0.0)
            e = np.exp(sc - mx)
            out[i, h] = (e / (math.exp(-mx) + e.sum())) @ v[lo:i + 1, g]
    return out


def mix_values(v, v_first, lam):
    """per token, over all value heads laid end to end"""
    return (1.0 - lam) * v + lam * v_first.reshape(v.shape)


def grouped_attention(h, W, p, m, eps, first_values):
    """first_values: None when this layer does not mix values; else a one-element list holding the first mixing layer's values (filled by that layer)"""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm((h @ W[p + ".q"].T).reshape(T, H, d), W[p + ".q.norm"], eps)
    k = rms_norm((h @ W[p + ".k"].T).reshape(T, G, d), W[p + ".k.norm"], eps)
    v = (h @ W[p + ".v"].T).reshape(T, G, dv)
    if first_values is not None:
        if not first_values:
            first_values.append(v)
        else:
            v = mix_values(v, first_values[0], float(W[p + ".vmix"]))
    a = chunked_bias_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size", 0))
    return a.reshape(T, H * dv) @ W[p + ".o"].T


# ---------------------------------------------------------------------------------------------------------------- feed-forward
def silu_expert(h, wg, wu, wd):
    g = h @ wg.T
    return (g / (1.0 + np.exp(-g)) * (h @ wu.T)) @ wd.T


def topk_router(h, wr, b, top):
    """ids [T, top] of the largest logits (lowest index among equals), weights = softmax over those logits only"""
    z = h @ wr.T + b
    ids = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zt = np.take_along_axis(z, ids, -1)
    e = np.exp(zt - zt.max(-1, keepdims=True))
    return ids, e / e.sum(-1, keepdims=True), z


def moe_ffn(h, W, p, mlp):
    ids, wts, _ = topk_router(h, W[p + ".router"], W[p + ".router.b"], mlp["router"]["top"])
    out = np.zeros((h.shape[0], W[p + ".e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, w in zip(ids[t], wts[t]):
            out[t] += w * silu_expert(h[t:t + 1], W[f"{p}.e{e}.gate"], W[f"{p}.e{e}.up"], W[f"{p}.e{e}.down"])[0]
    return out


# ---------------------------------------------------------------------------------------------------------------- the model
def forward(cfg, W32, tokens):
    """logits [T, vocab] and the residual stream after every layer [L, T, width], float64"""
    W = {k: np.asarray(v, np.float64) for k, v in W32.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    T = len(tokens)
    pos = np.arange(T)
    x = W["embed"][np.asarray(tokens)]
    first_values, streams = [], []
    for li, lc in enumerate(cfg["layers"]):
        p, m = f"l{li}", lc["mixer"]
        if lc["type"] == "latent_attention":
            y = latent_attention(x, W, p + ".mix", m, pos, eps)
        elif lc["type"] == "attention":
            y = grouped_attention(x, W, p + ".mix", m, eps, first_values if m.get("v_mix") else None)
        else:
            raise ValueError(lc["type"])
        x = x + mult * centered_norm(y, W[p + ".norm1"], eps)
        if lc.get("mlp") is not None:
            x = x + mult * centered_norm(moe_ffn(x, W, p + ".mlp", lc["mlp"]), W[p + ".norm2"], eps)
        streams.append(x.copy())
    return centered_norm(x, W["final.norm"], eps) @ W["head"].T, np.stack(streams)


# ---------------------------------------------------------------------------------------------------------------- random models
def make_config(width=96, vocab=101, eps=1e-5, residual_mult=0.7, layers=None):
    return {"architecture": "Pamulix", "layers": layers, "norm": {"eps": eps}, "residual_mult": residual_mult, "vocab": vocab, "width": width}


def attn(heads, kv_heads, dim, vdim, chunk, v_mix=False, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if chunk:
        m["mask"] = {"size": chunk}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, scaling=None, scale=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "rot": rot,
                                                   "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}}


def moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def layer(mixer, mlp):
    d = dict(mixer)
    d["mlp"] = mlp
    return d


def random_weights(cfg, seed=0, router_gain=4.0):
    """tensors by checkpoint name, float32 values that bfloat16 holds exactly (so a bf16 and an f32 store see the same model)"""
    rng = np.random.default_rng(seed)
    Wd, V = cfg["width"], cfg["vocab"]
    out = {}

    def mat(o, i, gain=1.0):
        return bf16_round((rng.standard_normal((o, i)) * gain / math.sqrt(i)).astype(np.float32))

    def vec(n, lo, hi):
        return bf16_round(rng.uniform(lo, hi, n).astype(np.float32))
    out["embed"] = bf16_round(rng.standard_normal((V, Wd)).astype(np.float32))
    out["head"] = mat(V, Wd)
    out["final.norm"] = vec(Wd, 0.5, 1.5)
    for li, lc in enumerate(cfg["layers"]):
        p, m = f"l{li}", lc["mixer"]
        out[p + ".norm1"] = vec(Wd, 0.5, 1.5)
        if lc["type"] == "attention":
            out[p + ".mix.q"] = mat(m["heads"] * m["dim"], Wd)
            out[p + ".mix.k"] = mat(m["kv_heads"] * m["dim"], Wd)
            out[p + ".mix.v"] = mat(m["kv_heads"] * m["vdim"], Wd)
            out[p + ".mix.q.norm"], out[p + ".mix.k.norm"] = vec(m["dim"], 0.5, 1.5), vec(m["dim"], 0.5, 1.5)
            if m.get("v_mix"):
                out[p + ".mix.vmix"] = bf16_round(np.asarray(rng.uniform(0.2, 0.8), np.float32))
            out[p + ".mix.o"] = mat(Wd, m["heads"] * m["vdim"])
        else:
            H, d, r = m["heads"], m["dim"], m["rot_dim"]
            out[p + ".mix.dq"], out[p + ".mix.dq.norm"] = mat(m["q_rank"], Wd), vec(m["q_rank"], 0.5, 1.5)
            out[p + ".mix.uq"] = mat(H * (d + r), m["q_rank"], 1.5)
            out[p + ".mix.dkv"], out[p + ".mix.dkv.norm"] = mat(m["kv_rank"] + r, Wd), vec(m["kv_rank"], 0.5, 1.5)
            out[p + ".mix.uk"], out[p + ".mix.uv"] = mat(H * d, m["kv_rank"], 1.5), mat(H * m["vdim"], m["kv_rank"])
            out[p + ".mix.o"] = mat(Wd, H * m["vdim"])
        mlp = lc.get("mlp")
        if mlp is None:
            continue
        out[p + ".norm2"] = vec(Wd, 0.5, 1.5)
        E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
        out[p + ".mlp.router"], out[p + ".mlp.router.b"] = mat(E, Wd, router_gain), vec(E, -1.0, 1.0)
        for e in range(E):
            out[f"{p}.mlp.e{e}.gate"], out[f"{p}.mlp.e{e}.up"], out[f"{p}.mlp.e{e}.down"] = mat(F, Wd, 2.0), mat(F, Wd, 2.0), mat(Wd, F)
    return out


def write_checkpoint(folder, cfg, weights):
    """config.json + model.safetensors (bfloat16 tensors) the way a checkpoint of the design is laid out"""
    import os
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, off = {}, [], 0
    for name, a in weights.items():
        b = to_bf16_bits(a).tobytes()
        header[name] = {"dtype": "BF16", "shape": list(np.shape(a)), "data_offsets": [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)
