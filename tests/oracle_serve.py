"""Plain, slow restatement of the layer-described Lomutar design in float64 numpy: one function per mechanism, the whole sequence at once, no cache.
It shares no code with the serving store; the tests compare the store's residual streams and logits with it.

Notation: x [T, width] residual stream; p [T] positions; for a head, q_i / k_j / v_j rows; W matrices are [out, in] and applied as x @ W.T."""
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


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / np.sqrt((x ** 2).mean(-1, keepdims=True) + eps)


def rotate_pairs(x, pos, dims, base, factor):
    """x [T, heads, dim]: coordinates (2i, 2i + 1), i < dims / 2, turn by the angle pos * base^(-2i / dims) / factor; the rest stays"""
    y = x.copy()
    for i in range(dims // 2):
        ang = pos.astype(np.float64) * (base ** (-2.0 * i / dims) / factor)
        c, s = np.cos(ang)[:, None], np.sin(ang)[:, None]
        a, b = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        y[:, :, 2 * i] = a * c - b * s
        y[:, :, 2 * i + 1] = b * c + a * s
    return y


def sink_window_attention(q, k, v, scale, window, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query i sees keys j with 0 <= i - j < window (window 0: all j <= i); weights =
    exp(score) / (sum of exp(score) over the visible keys + exp(sink_h))"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = 0 if window <= 0 else max(0, i - window + 1)
            sc = (k[lo:i + 1, g] @ q[i, h]) * scale
            m = max(sc.max(), sink[h]) if sink is not None else sc.max()
            e = np.exp(sc - m)
            den = e.sum() + (math.exp(sink[h] - m) if sink is not None else 0.0)
            out[i, h] = (e / den) @ v[lo:i + 1, g]
    return out


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def dense_ffn(h, wg, wu, wd):
    return (gelu_tanh(h @ wg.T) * (h @ wu.T)) @ wd.T


def clamped_expert(h, wg, wu, wd, limit):
    g = np.minimum(h @ wg.T, limit)
    u = np.clip(h @ wu.T, -limit, limit)
    return (g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0)) @ wd.T


def group_router(h, wr, top, groups, keep):
    """ids [T, top], weights [T, top]: softmax over all experts; the `keep` groups with the largest member score stay; the `top` largest scores among
    their experts; the weights are those scores as they are"""
    z = h @ wr.T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z)
    s /= s.sum(-1, keepdims=True)
    T, E = s.shape
    per = E // groups
    ids = np.zeros((T, top), np.int64)
    wts = np.zeros((T, top))
    for t in range(T):
        gs = s[t].reshape(groups, per).max(-1)
        kept = np.argsort(-gs, kind="stable")[:keep]
        allowed = np.zeros(E, bool)
        for g in kept:
            allowed[g * per:(g + 1) * per] = True
        cand = np.where(allowed, s[t], -1.0)
        ids[t] = np.argsort(-cand, kind="stable")[:top]
        wts[t] = s[t, ids[t]]
    return ids, wts, s


def moe_ffn(h, W, p, mlp):
    r = mlp["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    ids, wts, _ = group_router(h, W[p + ".router"], r["top"], g["count"], g["keep"])
    out = np.zeros((h.shape[0], W[p + ".e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, w in zip(ids[t], wts[t]):
            out[t] += w * clamped_expert(h[t:t + 1], W[f"{p}.e{e}.gate"], W[f"{p}.e{e}.up"], W[f"{p}.e{e}.down"], mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out += clamped_expert(h, W[p + ".shared.gate"], W[p + ".shared.up"], W[p + ".shared.down"], mlp["shared"]["limit"])
    return out


def forward(cfg, W32, tokens):
    """logits [T, vocab] and the residual stream after every layer [L, T, width], float64"""
    W = {k: np.asarray(v, np.float64) for k, v in W32.items()}
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    pos = np.arange(T)
    x = W["embed"][np.asarray(tokens)]
    cache, streams = {}, []
    for li, lc in enumerate(cfg["layers"]):
        p, m = f"l{li}", lc["mixer"]
        h = layer_norm(x, W[p + ".norm1"], W[p + ".norm1.b"], eps)
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        rot = m.get("rot")
        turn = (lambda a: rotate_pairs(a, pos, rot["dims"], rot["base"], (rot.get("scaling") or {}).get("factor", 1.0))) if rot else (lambda a: a)
        q = unit_rms(turn((h @ W[p + ".mix.q"].T).reshape(T, H, d)), eps)
        if m.get("kv_from") is not None:
            k, v = cache[m["kv_from"]]
        else:
            k = unit_rms(turn((h @ W[p + ".mix.k"].T).reshape(T, G, d)), eps)
            v = (h @ W[p + ".mix.v"].T).reshape(T, G, dv)
            cache[li] = (k, v)
        a = sink_window_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size", 0), W[p + ".mix.sink"])
        mix = a.reshape(T, H * dv) @ W[p + ".mix.o"].T
        mlp = lc.get("mlp")
        if mlp is None:
            ff = 0.0
        elif mlp["kind"] == "dense":
            ff = dense_ffn(h, W[p + ".mlp.gate"], W[p + ".mlp.up"], W[p + ".mlp.down"])
        else:
            ff = moe_ffn(h, W, p + ".mlp", mlp)
        x = x + (mix + ff)
        streams.append(x.copy())
    y = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return y @ W["head"].T, np.stack(streams)


# ---------------------------------------------------------------------------------------------------------------- random models
def make_config(width=96, vocab=101, eps=1e-5, layers=None):
    return {"architecture": "Lomutar", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def attn(heads, kv_heads, dim, vdim, window, rot_dims, base=10000.0, factor=1.0, scale=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims, "scaling": {"factor": factor}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, groups, keep, ff, limit, shared_ff=0, shared_limit=0.0):
    d = {"kind": "moe", "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}, "expert": {"ff": ff, "limit": limit}}
    if shared_ff:
        d["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return d


def random_weights(cfg, seed=0, router_gain=4.0, sink_range=(-1.0, 2.0)):
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
    out["final.norm"], out["final.norm.b"] = vec(Wd, 0.5, 1.5), vec(Wd, -0.2, 0.2)
    for li, lc in enumerate(cfg["layers"]):
        p, m = f"l{li}", lc["mixer"]
        out[p + ".norm1"], out[p + ".norm1.b"] = vec(Wd, 0.5, 1.5), vec(Wd, -0.2, 0.2)
        out[p + ".mix.q"] = mat(m["heads"] * m["dim"], Wd)
        if m.get("kv_from") is None:
            out[p + ".mix.k"] = mat(m["kv_heads"] * m["dim"], Wd)
            out[p + ".mix.v"] = mat(m["kv_heads"] * m["vdim"], Wd)
        out[p + ".mix.o"] = mat(Wd, m["heads"] * m["vdim"])
        out[p + ".mix.sink"] = vec(m["heads"], *sink_range)
        mlp = lc.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            out[p + ".mlp.gate"], out[p + ".mlp.up"], out[p + ".mlp.down"] = mat(mlp["ff"], Wd, 2.0), mat(mlp["ff"], Wd), mat(Wd, mlp["ff"])
        else:
            out[p + ".mlp.router"] = mat(mlp["router"]["experts"], Wd, router_gain)
            F = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                out[f"{p}.mlp.e{e}.gate"], out[f"{p}.mlp.e{e}.up"], out[f"{p}.mlp.e{e}.down"] = mat(F, Wd, 3.0), mat(F, Wd, 3.0), mat(Wd, F)
            if mlp.get("shared"):
                SF = mlp["shared"]["ff"]
                out[p + ".mlp.shared.gate"], out[p + ".mlp.shared.up"], out[p + ".mlp.shared.down"] = mat(SF, Wd, 3.0), mat(SF, Wd, 3.0), mat(Wd, SF)
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
        header[name] = {"dtype": "BF16", "shape": list(a.shape), "data_offsets": [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)
