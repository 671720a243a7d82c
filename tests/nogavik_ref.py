"""A plain, slow statement of the Nogavik design in numpy (float64): one function per mechanism, written from the design's equations and
sharing nothing with the product path.  The GPU tests compare the framework against it.

Notation: T tokens, E = width, H heads, G key heads, Dk per-head key size, Dv per-head value size, N state size of a state-space head.
Weights are [out, in] and applied as W @ x.  A model is (cfg, W): cfg is the parsed config.json, W maps tensor names to float64 arrays.
Every sequence starts at position 0 with every state at zero."""
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


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def norm_one_plus(x, w, eps):
    """the model's norm: the weight is stored around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def short_conv(u, w, bias=None):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] * u_{t - taps + 1 + j} (+ bias); what lies before the start is zero."""
    T, taps = u.shape[0], w.shape[1]
    pad = np.concatenate([np.zeros((taps - 1, u.shape[1])), u], axis=0)
    y = np.zeros_like(u)
    for j in range(taps):
        y += pad[j:j + T] * w[:, j]
    return y if bias is None else y + bias


def rotate_pairs(x, pos, dims, base):
    """x [T, heads, D]: entries 2i and 2i + 1 (i < dims / 2) of a head turn by pos * base^(-2i / dims); entries from dims on pass unchanged."""
    half = dims // 2
    f = np.asarray([float(base) ** (-2.0 * i / dims) for i in range(half)])
    a = np.asarray(pos, dtype=np.float64)[:, None, None] * f[None, None, :]
    c, s = np.cos(a), np.sin(a)
    out = x.copy()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def causal_softmax_attention(q, k, v, scale):
    """q [T, H, Dk], k [T, G, Dk], v [T, G, Dv] -> [T, H, Dv]; query head h reads key head h // (H / G); position i sees j <= i."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = np.where(np.tril(np.ones((T, T), dtype=bool)), s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ v[:, g]
    return out


# ---------------------------------------------------------------------------------------------------------------- recurrences, token by token
def delta_rule_channel_decay(q, k, v, beta, decay):
    """q, k [T, G, Dk] (already unit vectors, q scaled); v [T, H, Dv]; beta [T, H]; decay [T, H, Dk] -> [T, H, Dv].
    Per head, S [Dk, Dv] from zero: S <- diag(decay) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, Dv = v.shape
    G, Dk = k.shape[1], k.shape[2]
    o = np.zeros((T, H, Dv))
    for h in range(H):
        g = h // (H // G)
        S = np.zeros((Dk, Dv))
        for t in range(T):
            S = decay[t, h][:, None] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, g])
            S = S + np.outer(k[t, g], u)
            o[t, h] = S.T @ q[t, g]
    return o


def state_space_scan(x, B, C, dt, A, D):
    """x [T, H, Dv]; B, C [T, G, N]; dt [T, H] (after softplus); A [H] (= exp(A_log)); D [H] -> [T, H, Dv].
    Per head, S [N, Dv] from zero: S <- exp(-A dt) S + dt B x^T; y = S^T C + D x."""
    T, H, Dv = x.shape
    G, N = B.shape[1], B.shape[2]
    y = np.zeros((T, H, Dv))
    for h in range(H):
        g = h // (H // G)
        S = np.zeros((N, Dv))
        for t in range(T):
            S = math.exp(-A[h] * dt[t, h]) * S + dt[t, h] * np.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + D[h] * x[t, h]
    return y


# ---------------------------------------------------------------------------------------------------------------- mixers
def mixer_latent(h, pos, mx, W, p, eps, shared=None):
    """latent attention; returns (output [T, E], (latent c [T, R], rotated key part [T, Dr])) — the pair is what a layer with kv_from re-uses."""
    H, Dk, Dr, Dv = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"]
    T = h.shape[0]
    cq = rms_unit(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).reshape(T, H, Dk + Dr)
    if shared is None:
        ckr = h @ W[p + "dkv"].T
        R = ckr.shape[1] - Dr
        c = rms_unit(ckr[:, :R], eps) * W[p + "dkv.norm"]
        kr = rotate_pairs(ckr[:, None, R:], pos, mx["rot"]["dims"], mx["rot"]["base"])[:, 0] if Dr > 0 else ckr[:, R:]
    else:
        c, kr = shared
    qn = q[..., :Dk]
    qr = rotate_pairs(q[..., Dk:], pos, mx["rot"]["dims"], mx["rot"]["base"]) if Dr > 0 else q[..., Dk:]
    kn = (c @ W[p + "uk"].T).reshape(T, H, Dk)
    vv = (c @ W[p + "uv"].T).reshape(T, H, Dv)
    kfull = np.concatenate([kn, np.repeat(kr[:, None, :], H, axis=1)], axis=2)
    o = causal_softmax_attention(np.concatenate([qn, qr], axis=2), kfull, vv, mx["scale"]).reshape(T, H * Dv)
    o = o * sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T, (c, kr)


def mixer_state_space(h, mx, W, p, eps):
    H, Dv, N, G, ng = mx["heads"], mx["vdim"], mx["state"], mx["groups"], mx["norm_groups"]
    T, inner = h.shape[0], mx["heads"] * mx["vdim"]
    u = h @ W[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, Dv)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + W[p + "dt_bias"])
    y = state_space_scan(x, B, C, dt, np.exp(W[p + "A_log"]), W[p + "D"]).reshape(T, inner)
    y = y * silu(z)
    y = rms_unit(y.reshape(T, ng, inner // ng), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def mixer_parallel_left(h, mx, W, p, eps):
    H, G, Dk, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).reshape(T, H, Dk)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).reshape(T, G, Dk)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).reshape(T, G, Dv)
    q = rms_unit(q, eps) * W[p + "q.norm"]
    k = rms_unit(k, eps) * W[p + "k.norm"]
    return causal_softmax_attention(q, k, v, mx["scale"]).reshape(T, H * Dv) @ W[p + "o"].T


def mixer_parallel_right(h, mx, W, p, eps):
    H, G, Dk, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    q = silu(short_conv(h @ W[p + "q"].T, W[p + "q.conv"])).reshape(T, G, Dk)
    k = silu(short_conv(h @ W[p + "k"].T, W[p + "k.conv"])).reshape(T, G, Dk)
    v = silu(short_conv(h @ W[p + "v"].T, W[p + "v.conv"])).reshape(T, H, Dv)
    q = q / np.sqrt((q * q).sum(axis=-1, keepdims=True) + 1e-6) * Dk ** -0.5
    k = k / np.sqrt((k * k).sum(axis=-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ W[p + "b"].T)
    a = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]
    decay = np.exp(-np.exp(W[p + "A_log"])[None, :, None] * softplus(a).reshape(T, H, Dk))
    o = delta_rule_channel_decay(q, k, v, beta, decay)
    o = rms_unit(o, eps) * W[p + "norm"]
    o = o.reshape(T, H * Dv) * sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T)
    return o @ W[p + "o"].T


def mixer_parallel(h, mx, W, p, eps):
    left = mixer_parallel_left(h, mx["left"], W, p + "left.", eps)
    right = mixer_parallel_right(h, mx["right"], W, p + "right.", eps)
    return 0.5 * (rms_unit(left, eps) * W[p + "left.out"] + rms_unit(right, eps) * W[p + "right.out"])


def feed_forward(h, W, p):
    return np.maximum(h @ W[p + "up"].T, 0.0) ** 2 @ W[p + "down"].T


def token_side(x, tokens, il, cfg, W, eps):
    """the per-layer token input: layer il's part of the side table, gated by the stream, projected back, normed and added."""
    d = cfg["token_side"]["dim"]
    p = "l%d.side." % il
    e = W["side.embed"][np.asarray(tokens), il * d:(il + 1) * d]
    y = (gelu_tanh(x @ W[p + "gate"].T) * e) @ W[p + "proj"].T
    return x + rms_unit(y, eps) * W[p + "norm"]


# ---------------------------------------------------------------------------------------------------------------- the model
def forward(cfg, W, tokens, residuals=None):
    """logits [T, vocab] of one sequence from position 0; `residuals` (a list) receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    pos = np.arange(T)
    x = W["embed"][np.asarray(tokens)]
    kept = {}
    for il, L in enumerate(cfg["layers"]):
        p, mx = "l%d." % il, L["mixer"]
        h = norm_one_plus(x, W[p + "norm1"], eps)
        if L["type"] == "latent_attention":
            m, kept[il] = mixer_latent(h, pos, mx, W, p + "mix.", eps, kept[mx["kv_from"]] if mx.get("kv_from") is not None else None)
        elif L["type"] == "mamba2":
            m = mixer_state_space(h, mx, W, p + "mix.", eps)
        elif L["type"] == "parallel":
            m = mixer_parallel(h, mx, W, p + "mix.", eps)
        else:
            raise ValueError("unknown mixer " + L["type"])
        if L.get("mlp"):
            m = m + feed_forward(norm_one_plus(x, W[p + "norm2"], eps), W, p + "mlp.")
        x = x + m
        if cfg.get("token_side"):
            x = token_side(x, tokens, il, cfg, W, eps)
        if residuals is not None:
            residuals.append(x.copy())
    return norm_one_plus(x, W["final.norm"], eps) @ W["embed"].T


# ---------------------------------------------------------------------------------------------------------------- making models
def bf16_round(a):
    """float array -> the nearest bfloat16 values (round to nearest even), as float64."""
    b = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16 << 16).astype(np.uint32)
    return b.view(np.float32).astype(np.float64)


def tensor_shapes(cfg):
    E, V = cfg["width"], cfg["vocab"]
    sh = {"embed": (V, E), "final.norm": (E,)}
    side = cfg.get("token_side")
    if side:
        sh["side.embed"] = (V, side["dim"] * len(cfg["layers"]))
    for il, L in enumerate(cfg["layers"]):
        p, mx = "l%d." % il, L["mixer"]
        m = p + "mix."
        sh[p + "norm1"] = (E,)
        if L["type"] == "latent_attention":
            H, Dk, Dr, Dv, R, Rq = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"], mx["q_rank"]
            sh.update({m + "dq": (Rq, E), m + "dq.norm": (Rq,), m + "uq": (H * (Dk + Dr), Rq), m + "uk": (H * Dk, R), m + "uv": (H * Dv, R),
                       m + "g": (H * Dv, E), m + "o": (E, H * Dv)})
            if mx.get("kv_from") is None:
                sh.update({m + "dkv": (R + Dr, E), m + "dkv.norm": (R,)})
        elif L["type"] == "mamba2":
            H, Dv, N, G, taps = mx["heads"], mx["vdim"], mx["state"], mx["groups"], mx["conv"]
            inner, ch = H * Dv, H * Dv + 2 * G * N
            sh.update({m + "in": (2 * inner + 2 * G * N + H, E), m + "conv": (ch, taps), m + "conv.b": (ch,), m + "dt_bias": (H,), m + "A_log": (H,),
                       m + "D": (H,), m + "norm": (inner,), m + "o": (E, inner)})
        else:
            a, r = mx["left"], mx["right"]
            H, G, Dk, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            l_ = m + "left."
            sh.update({l_ + "q": (H * Dk, E), l_ + "q.b": (H * Dk,), l_ + "k": (G * Dk, E), l_ + "k.b": (G * Dk,), l_ + "v": (G * Dv, E),
                       l_ + "v.b": (G * Dv,), l_ + "q.norm": (Dk,), l_ + "k.norm": (Dk,), l_ + "o": (E, H * Dv), l_ + "out": (E,)})
            H, G, Dk, Dv, taps, rank = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"], r.get("rank", 8)
            r_ = m + "right."
            sh.update({r_ + "q": (G * Dk, E), r_ + "q.conv": (G * Dk, taps), r_ + "k": (G * Dk, E), r_ + "k.conv": (G * Dk, taps),
                       r_ + "v": (H * Dv, E), r_ + "v.conv": (H * Dv, taps), r_ + "b": (H, E), r_ + "A_log": (H,), r_ + "norm": (Dv,),
                       r_ + "a1": (rank, E), r_ + "a2": (H * Dk, rank), r_ + "dt_bias": (H * Dk,), r_ + "g1": (rank, E), r_ + "g2": (H * Dv, rank),
                       r_ + "o": (E, H * Dv), r_ + "out": (E,)})
        if L.get("mlp"):
            sh.update({p + "norm2": (E,), p + "mlp.up": (L["mlp"]["ff"], E), p + "mlp.down": (E, L["mlp"]["ff"])})
        if side:
            sh.update({p + "side.gate": (side["dim"], E), p + "side.proj": (E, side["dim"]), p + "side.norm": (E,)})
    return sh


def random_weights(cfg, seed):
    """bf16-representable random weights with magnitudes that keep every mechanism alive (decays away from 0 and 1, gates that move)."""
    rng = np.random.default_rng(seed)
    W = {}
    for name, s in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2") or name == "final.norm":
            a = rng.normal(0, 0.2, s)          # stored around zero: the norm multiplies by 1 + w
        elif leaf in ("norm", "out"):
            a = rng.uniform(0.7, 1.4, s)
        elif leaf == "conv":
            a = rng.normal(0, 0.5, s)
        elif leaf == "A_log":
            a = rng.uniform(-2.0, 0.5, s)
        elif leaf == "dt_bias":
            a = rng.uniform(-1.0, 1.0, s)
        elif leaf == "D":
            a = rng.normal(0, 1.0, s)
        elif leaf == "b" and len(s) == 1:
            a = rng.normal(0, 0.3, s)
        elif name in ("embed", "side.embed"):
            a = rng.normal(0, 1.0, s)
        elif leaf in ("a2", "g2"):
            a = rng.normal(0, 2.0 / math.sqrt(s[-1]), s)
        else:
            a = rng.normal(0, 1.0 / math.sqrt(s[-1]), s)
        W[name] = bf16_round(a)
    return W


def dense(ff):
    return {"kind": "dense", "ff": ff}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, mlp, base=10000.0, kv_from=None):
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
          "rot": {"dims": rot_dim, "base": base}}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mx, "mlp": mlp}


def state_space_layer(heads, vdim, state, groups, norm_groups, conv, mlp):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}, "mlp": mlp}


def parallel_layer(heads, kv_heads, dim, vdim, scale, r_heads, r_kv_heads, r_dim, r_vdim, conv, mlp, rank=8):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    right = {"heads": r_heads, "kv_heads": r_kv_heads, "dim": r_dim, "vdim": r_vdim, "conv": conv, "rank": rank}
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def make_config(width, vocab, layers, side_dim=8, eps=1e-5):
    cfg = {"architecture": "Nogavik", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if side_dim:
        cfg["token_side"] = {"dim": side_dim}
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
