"""A plain, slow statement of the Rarelorn design in numpy (float64): one function per mechanism, written from the design's equations and
sharing nothing with the product path.  The GPU tests compare the framework against it.

Notation: T tokens, E = width, H heads, G key heads, Dk per-head key size, Dv per-head value size.  Weights are [out, in] and applied as
W @ x.  A model is (cfg, W): cfg is the parsed config.json, W maps tensor names to float64 arrays.  Every sequence starts at position 0
with every state at zero."""
import json
import math
import os
import struct

import numpy as np


# ---------------------------------------------------------------------------------------------------------------- small pieces
def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def short_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] * u_{t - taps + 1 + j}; what lies before the start is zero."""
    T, taps = u.shape[0], w.shape[1]
    pad = np.concatenate([np.zeros((taps - 1, u.shape[1])), u], axis=0)
    y = np.zeros_like(u)
    for j in range(taps):
        y += pad[j:j + T] * w[:, j]
    return y


def rotate_half(x, pos, dims, base):
    """x [T, heads, D]: entry i < dims/2 of a head is paired with entry i + dims/2; entries from dims on pass unchanged."""
    half = dims // 2
    f = np.asarray([float(base) ** (-2.0 * i / dims) for i in range(half)])
    a = np.asarray(pos, dtype=np.float64)[:, None, None] * f[None, None, :]
    c, s = np.cos(a), np.sin(a)
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def window_visible(T, size):
    """[T, T] bool: i sees j when 0 <= i - j < size."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & (i - j < size)


def token_shift_mix(h, mu):
    """h [T, E] of one sequence from its start: h_t + (h_{t-1} - h_t) * mu with h_{-1} = 0."""
    prev = np.concatenate([np.zeros_like(h[:1]), h[:-1]], axis=0)
    return h + (prev - h) * mu


# ---------------------------------------------------------------------------------------------------------------- mixers
def delta_mixer(h, W, p, mx, eps):
    """Gated delta rule: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, Dk, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = silu(short_conv(h @ W[p + "q"].T, W[p + "q.conv"])).reshape(T, G, Dk)
    k = silu(short_conv(h @ W[p + "k"].T, W[p + "k.conv"])).reshape(T, G, Dk)
    v = silu(short_conv(h @ W[p + "v"].T, W[p + "v.conv"])).reshape(T, H, Dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * Dk ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ W[p + "b"].T)
    g = np.exp(-np.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    gate = silu(h @ W[p + "g"].T).reshape(T, H, Dv)
    o = np.zeros((T, H, Dv))
    for hd in range(H):
        kh = hd // (H // G)
        S = np.zeros((Dk, Dv))
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kh])
            S = S + np.outer(k[t, kh], u)
            o[t, hd] = S.T @ q[t, kh]
    o = rms_unit(o, eps) * W[p + "norm"] * gate
    return o.reshape(T, H * Dv) @ W[p + "o"].T


def sigmoid_attention(h, W, p, mx):
    """Windowed attention whose weights are sigmoid(capped score + bias): no normalisation over the keys."""
    T = h.shape[0]
    H, G, Dk, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = short_conv(h @ W[p + "q"].T + W[p + "q.b"], W[p + "q.conv"]).reshape(T, H, Dk)
    k = short_conv(h @ W[p + "k"].T + W[p + "k.b"], W[p + "k.conv"]).reshape(T, G, Dk)
    v = short_conv(h @ W[p + "v"].T + W[p + "v.b"], W[p + "v.conv"]).reshape(T, G, Dv)
    pos = np.arange(T)
    rot = mx.get("rot")
    if rot and rot["dims"]:
        q = rotate_half(q, pos, rot["dims"], rot["base"])
        k = rotate_half(k, pos, rot["dims"], rot["base"])
    ok = window_visible(T, mx["mask"]["size"])
    cap = mx["softcap"]
    out = np.zeros((T, H, Dv))
    for hd in range(H):
        kh = hd // (H // G)
        s = (q[:, hd] @ k[:, kh].T) * mx["scale"] * W[p + "temp"][hd]
        if cap:  # (0: scores are not capped)
            s = cap * np.tanh(s / cap)
        w = np.where(ok, sigmoid(s + W[p + "pb"][hd]), 0.0)
        out[:, hd] = w @ v[:, kh]
    return out.reshape(T, H * Dv) @ W[p + "o"].T + W[p + "o.b"]


def time_mix(h, W, p, mx, eps):
    """RWKV-style time mixing with a data-dependent decay per key channel and a bonus for the current token."""
    T = h.shape[0]
    H, D = mx["heads"], mx["dim"]
    mix = {s: token_shift_mix(h, W[p + "mu." + s]) for s in "rkvgw"}
    r = (mix["r"] @ W[p + "r"].T).reshape(T, H, D)
    k = (mix["k"] @ W[p + "k"].T).reshape(T, H, D)
    v = (mix["v"] @ W[p + "v"].T).reshape(T, H, D)
    gate = silu(mix["g"] @ W[p + "g"].T)
    w = np.exp(-np.exp(np.tanh(mix["w"] @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])).reshape(T, H, D)
    u = W[p + "u"].reshape(H, D)
    o = np.zeros((T, H, D))
    for hd in range(H):
        S = np.zeros((D, D))
        for t in range(T):
            kv = np.outer(k[t, hd], v[t, hd])
            o[t, hd] = (S + u[hd][:, None] * kv).T @ r[t, hd]
            S = w[t, hd][:, None] * S + kv
    o = rms_unit(o, eps).reshape(T, H * D) * W[p + "norm"] * gate
    return o @ W[p + "o"].T


def parallel_mixer(h, W, p, mx, eps):
    left = sigmoid_attention(h, W, p + "left.", mx["left"])
    right = time_mix(h, W, p + "right.", mx["right"], eps)
    return mx["left_scale"] * left + mx["right_scale"] * right


def mlstm_mixer(h, W, p, mx, eps):
    """Matrix memory with exponential gates kept in range by a running maximum m (m starts at 0)."""
    T = h.shape[0]
    H, Dk, Dv, cap = mx["heads"], mx["dim"], mx["vdim"], mx["gate_cap"]
    q = (h @ W[p + "q"].T).reshape(T, H, Dk) * Dk ** -0.5
    k = (h @ W[p + "k"].T).reshape(T, H, Dk)
    v = (h @ W[p + "v"].T).reshape(T, H, Dv)
    ig = cap * np.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    fg = log_sigmoid(cap * np.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    o = np.zeros((T, H, Dv))
    for hd in range(H):
        S, n, m = np.zeros((Dk, Dv)), np.zeros(Dk), 0.0
        for t in range(T):
            m_new = max(fg[t, hd] + m, ig[t, hd])
            a, b = math.exp(fg[t, hd] + m - m_new), math.exp(ig[t, hd] - m_new)
            S = a * S + b * np.outer(k[t, hd], v[t, hd])
            n = a * n + b * k[t, hd]
            m = m_new
            o[t, hd] = S.T @ q[t, hd] / (max(abs(n @ q[t, hd]), math.exp(-m)) + 1e-6)
    o = rms_unit(o, eps).reshape(T, H * Dv) * W[p + "norm"] * sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


MIXERS = {"delta": delta_mixer, "parallel": parallel_mixer, "mlstm": mlstm_mixer}


# ---------------------------------------------------------------------------------------------------------------- feed-forward
def router_choice(z, r):
    """z [T, experts] logits -> (chosen [T, top], weights [T, top]): soft-max over all experts, choice confined to the best groups."""
    E, top = r["experts"], r["top"]
    s = np.exp(z - z.max(-1, keepdims=True))
    s = s / s.sum(-1, keepdims=True)
    allowed = np.ones_like(s, dtype=bool)
    gr = r.get("groups")
    if gr and gr["count"] > 1 and gr["keep"] < gr["count"]:
        per = E // gr["count"]
        best = s.reshape(-1, gr["count"], per).max(-1)
        order = np.argsort(-best, axis=-1, kind="stable")[:, :gr["keep"]]
        allowed[:] = False
        for t in range(s.shape[0]):
            for g in order[t]:
                allowed[t, g * per:(g + 1) * per] = True
    chosen = np.argsort(-np.where(allowed, s, -1.0), axis=-1, kind="stable")[:, :top]
    return chosen, np.take_along_axis(s, chosen, axis=-1) * r["scale"]


def moe(h, W, p, ff):
    r = ff["router"]
    chosen, wts = router_choice(h @ W[p + "router"].T, r)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t], wts[t]):
            pe = "%se%d." % (p, e)
            out[t] += w * ((silu(W[pe + "gate"] @ h[t]) * (W[pe + "up"] @ h[t])) @ W[pe + "down"].T)
    return out


# ---------------------------------------------------------------------------------------------------------------- the model
def layer(x, cfg, W, il):
    L, eps, p = cfg["layers"][il], cfg["norm"]["eps"], "l%d." % il
    x = x + MIXERS[L["type"]](rms_unit(x, eps) * W[p + "norm1"], W, p + "mix.", L["mixer"], eps)
    if L.get("mlp"):
        x = x + moe(rms_unit(x, eps) * W[p + "norm2"], W, p + "mlp.", L["mlp"])
    return x


def layer_runs(cfg):
    """[(layer, pass, first of its pass)] in the order of execution."""
    n, lp = len(cfg["layers"]), cfg.get("loop")
    if not lp:
        return [(i, 0, False) for i in range(n)]
    runs = [(i, 0, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        runs += [(i, t, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, 0, False) for i in range(lp["stop"], n)]


def forward(cfg, W, tokens, residuals=None):
    """logits [T, vocab] of ONE sequence from its start; residuals (a list) receives x after every layer run."""
    x = e0 = W["embed"][np.asarray(tokens)]
    for il, t, first in layer_runs(cfg):
        if first:
            if t > 0:
                x = x + e0
            x = x + W["loop.step"][t]
        x = layer(x, cfg, W, il)
        if residuals is not None:
            residuals.append(x.copy())
    return (rms_unit(x, cfg["norm"]["eps"]) * W["final.norm"]) @ W["head"].T


# ---------------------------------------------------------------------------------------------------------------- making models
def bf16_round(a):
    """float array -> the nearest bfloat16 values (round to nearest even), as float64."""
    b = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16 << 16).astype(np.uint32)
    return b.view(np.float32).astype(np.float64)


def tensor_shapes(cfg):
    E, V = cfg["width"], cfg["vocab"]
    sh = {"embed": (V, E), "head": (V, E), "final.norm": ()}
    if cfg.get("loop"):
        sh["loop.step"] = (cfg["loop"]["times"], E)
    for il, L in enumerate(cfg["layers"]):
        p, mx = "l%d." % il, L["mixer"]
        sh[p + "norm1"] = ()
        m = p + "mix."
        if L["type"] == "mlstm":
            H, Dk, Dv = mx["heads"], mx["dim"], mx["vdim"]
            sh.update({m + "q": (H * Dk, E), m + "k": (H * Dk, E), m + "v": (H * Dv, E), m + "g": (H * Dv, E), m + "o": (E, H * Dv),
                       m + "norm": (H * Dv,), m + "i": (H, E), m + "i.b": (H,), m + "f": (H, E), m + "f.b": (H,)})
        elif L["type"] == "delta":
            H, G, Dk, Dv, taps = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"], mx["conv"]
            sh.update({m + "q": (G * Dk, E), m + "q.conv": (G * Dk, taps), m + "k": (G * Dk, E), m + "k.conv": (G * Dk, taps),
                       m + "v": (H * Dv, E), m + "v.conv": (H * Dv, taps), m + "b": (H, E), m + "A_log": (H,), m + "norm": (Dv,),
                       m + "a": (H, E), m + "dt_bias": (H,), m + "g": (H * Dv, E), m + "o": (E, H * Dv)})
        else:
            a, r = mx["left"], mx["right"]
            H, G, Dk, Dv, taps = a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["conv"]
            l_ = m + "left."
            sh.update({l_ + "q": (H * Dk, E), l_ + "q.b": (H * Dk,), l_ + "k": (G * Dk, E), l_ + "k.b": (G * Dk,), l_ + "v": (G * Dv, E),
                       l_ + "v.b": (G * Dv,), l_ + "q.conv": (H * Dk, taps), l_ + "k.conv": (G * Dk, taps), l_ + "v.conv": (G * Dv, taps),
                       l_ + "temp": (H,), l_ + "pb": (H,), l_ + "o": (E, H * Dv), l_ + "o.b": (E,)})
            r_, C = m + "right.", r["heads"] * r["dim"]
            rank = r.get("rank", 8)
            for s in "rkvgw":
                sh[r_ + "mu." + s] = (E,)
            sh.update({r_ + "r": (C, E), r_ + "k": (C, E), r_ + "v": (C, E), r_ + "g": (C, E), r_ + "w1": (rank, E), r_ + "w2": (C, rank),
                       r_ + "w0": (C,), r_ + "u": (r["heads"], r["dim"]), r_ + "norm": (C,), r_ + "o": (E, C)})
        if L.get("mlp"):
            sh[p + "norm2"] = ()
            f = p + "mlp."
            sh[f + "router"] = (L["mlp"]["router"]["experts"], E)
            for e in range(L["mlp"]["router"]["experts"]):
                sh.update({"%se%d.gate" % (f, e): (L["mlp"]["expert"]["ff"], E), "%se%d.up" % (f, e): (L["mlp"]["expert"]["ff"], E),
                           "%se%d.down" % (f, e): (E, L["mlp"]["expert"]["ff"])})
    return sh


def random_weights(cfg, seed):
    """bf16-representable random weights with magnitudes that keep every mechanism alive (decays away from 0 and 1, gates that move)."""
    rng = np.random.default_rng(seed)
    W = {}
    for name, s in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if name.endswith("norm1") or name.endswith("norm2") or name == "final.norm":
            a = rng.uniform(0.8, 1.3, s)
        elif leaf == "norm":
            a = rng.uniform(0.7, 1.4, s)
        elif leaf == "conv":
            a = rng.normal(0, 0.5, s)
        elif ".mu." in name:
            a = rng.uniform(0.05, 0.95, s)
        elif leaf == "A_log":
            a = rng.uniform(-2.0, 0.5, s)
        elif leaf == "dt_bias":
            a = rng.uniform(-1.0, 1.0, s)
        elif leaf == "w0":
            a = rng.uniform(-3.0, 0.0, s)
        elif leaf == "u":
            a = rng.normal(0, 0.5, s)
        elif leaf == "temp":
            a = rng.uniform(0.6, 1.6, s)
        elif leaf == "pb":
            a = rng.uniform(-3.0, -1.0, s)
        elif leaf == "b" and len(s) == 1:
            a = rng.normal(0, 0.3, s)
        elif name in ("embed", "loop.step"):
            a = rng.normal(0, 1.0, s)
        elif leaf in ("i", "f"):
            a = rng.normal(0, 2.0 / math.sqrt(s[-1]), s)
        elif leaf == "router":
            a = rng.normal(0, 3.0 / math.sqrt(s[-1]), s)
        else:
            a = rng.normal(0, 1.0 / math.sqrt(s[-1]), s)
        W[name] = bf16_round(a)
    return W


def moe_cfg(ff, experts, top, count=1, keep=1, scale=1.0):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}


def mlstm_layer(heads, dim, vdim, mlp, gate_cap=15.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}, "mlp": mlp}


def delta_layer(heads, kv_heads, dim, vdim, conv, mlp):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def parallel_layer(heads, kv_heads, dim, vdim, conv, size, rot_dims, scale, softcap, r_heads, r_dim, mlp, base=10000.0, left_scale=1.0,
                   right_scale=1.0, rank=8):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "mask": {"size": size},
            "rot": {"dims": rot_dims, "base": base}, "scale": scale, "softcap": softcap}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": r_heads, "dim": r_dim, "rank": rank}, "left_scale": left_scale,
                                          "right_scale": right_scale}, "mlp": mlp}


def make_config(width, vocab, layers, loop=None, eps=1e-5):
    cfg = {"architecture": "Rarelorn", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def save_model(cfg, W, folder):
    """config.json (the helper key 'rank' is left out: the tensors' shapes give it) + model.safetensors with every tensor as bf16."""
    os.makedirs(folder, exist_ok=True)
    out = json.loads(json.dumps(cfg))
    for L in out["layers"]:
        if L["type"] == "parallel":
            L["mixer"]["right"].pop("rank", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(out, f)
    head, blobs, at = {}, [], 0
    for name, a in W.items():
        b = (np.asarray(a, dtype=np.float32).view(np.uint32) >> 16).astype("<u2").tobytes()
        head[name] = {"dtype": "BF16", "shape": list(np.shape(a)), "data_offsets": [at, at + len(b)]}
        blobs.append(b)
        at += len(b)
    hj = json.dumps(head).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))
