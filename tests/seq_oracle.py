"""Plain, slow float64 statement of the layer-list design (checker only: it shares no code with powerserve_amd).

Everything is computed for a whole sequence at once with explicit loops over time; one function per mechanism.  W maps tensor names to
float arrays, cfg is the parsed config.json.  Notation: x residual stream [T, width]; h what a sublayer reads; S a recurrent state.
"""
import numpy as np


def unit_rms(a, eps):
    return a / np.sqrt(np.mean(a * a, axis=-1, keepdims=True) + eps)


def offset_norm(a, w, eps):
    """RMS norm whose stored weight is the deviation from one."""
    return unit_rms(a, eps) * (1.0 + w)


def silu(a):
    return a / (1.0 + np.exp(-a))


def softplus(a):
    return np.logaddexp(0.0, a)


def time_conv(a, w):
    """Per-channel causal filter: out[t] = sum_j w[:, j] * a[t - (taps - 1) + j], nothing before t = 0.  a [T, C], w [C, taps]."""
    T, taps = a.shape[0], w.shape[1]
    out = np.zeros_like(a)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                out[t] += w[:, j] * a[s]
    return out


def xielu(z, p, q):
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (np.expm1(np.minimum(z, 0.0)) - z) + 0.5 * z
    return np.where(z > 0, pos, neg)


def wkv_mixer(W, pre, h, mc, eps):
    T, width = h.shape
    H, d = mc["heads"], mc["dim"]
    out = np.zeros((T, H * d))
    S = np.zeros((H, d, d))
    prev = np.zeros(width)
    bonus = W[pre + "u"]
    for t in range(T):
        mixed = {s: h[t] + (prev - h[t]) * W[pre + "mu." + s] for s in "rkvgw"}
        r = (W[pre + "r"] @ mixed["r"]).reshape(H, d)
        k = (W[pre + "k"] @ mixed["k"]).reshape(H, d)
        v = (W[pre + "v"] @ mixed["v"]).reshape(H, d)
        gate = silu(W[pre + "g"] @ mixed["g"])
        decay = np.exp(-np.exp(W[pre + "w2"] @ np.tanh(W[pre + "w1"] @ mixed["w"]) + W[pre + "w0"])).reshape(H, d)
        o = np.zeros((H, d))
        for hd in range(H):
            kv = np.outer(k[hd], v[hd])
            o[hd] = (S[hd] + bonus[hd][:, None] * kv).T @ r[hd]
            S[hd] = decay[hd][:, None] * S[hd] + kv
        out[t] = unit_rms(o, eps).reshape(-1) * W[pre + "norm"] * gate
        prev = h[t]
    return out @ W[pre + "o"].T


def delta_mixer(W, pre, h, mc, eps):
    T = h.shape[0]
    H, KH, d, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]

    def branch(name):
        return silu(time_conv(h @ W[pre + name].T, W[pre + name + ".conv"]))

    q, k, v = branch("q").reshape(T, KH, d), branch("k").reshape(T, KH, d), branch("v").reshape(T, H, dv)
    q = q / np.sqrt(np.sum(q * q, -1, keepdims=True) + 1e-6) / np.sqrt(d)
    k = k / np.sqrt(np.sum(k * k, -1, keepdims=True) + 1e-6)
    beta = 1.0 / (1.0 + np.exp(-(h @ W[pre + "b"].T)))
    keep = np.exp(-np.exp(W[pre + "A_log"]) * softplus(h @ W[pre + "a"].T + W[pre + "dt_bias"]))
    gate = silu(h @ W[pre + "g"].T).reshape(T, H, dv)
    S = np.zeros((H, d, dv))
    out = np.zeros((T, H, dv))
    for t in range(T):
        for hd in range(H):
            g = hd // (H // KH)
            S[hd] *= keep[t, hd]
            write = beta[t, hd] * (v[t, hd] - S[hd].T @ k[t, g])
            S[hd] += np.outer(k[t, g], write)
            out[t, hd] = S[hd].T @ q[t, g]
    out = unit_rms(out, eps) * W[pre + "norm"] * gate
    return out.reshape(T, H * dv) @ W[pre + "o"].T


def rotate(vec, pos, base, dims):
    """First `dims` numbers of vec turn in pairs (i, i + dims/2) by pos * base^(-2i/dims); the rest is kept."""
    out = np.array(vec, dtype=np.float64)
    half = dims // 2
    for i in range(half):
        ang = pos * base ** (-2.0 * i / dims)
        a, b = vec[..., i], vec[..., i + half]
        out[..., i] = a * np.cos(ang) - b * np.sin(ang)
        out[..., i + half] = b * np.cos(ang) + a * np.sin(ang)
    return out


def latent_mixer(W, pre, h, mc, eps, window=None):
    T = h.shape[0]
    H, d, dr, dv, R = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    window = mc["mask"]["size"] if window is None else window
    base, dims = mc["rot"]["base"], mc["rot"]["dims"]
    out = np.zeros((T, H * dv))
    lat, shared = [], []
    for t in range(T):
        both = W[pre + "dkv"] @ h[t]
        lat.append(unit_rms(both[:R], eps) * W[pre + "dkv.norm"])
        shared.append(rotate(both[R:], t, base, dims))
        cq = unit_rms(W[pre + "dq"] @ h[t], eps) * W[pre + "dq.norm"]
        q = (W[pre + "uq"] @ cq).reshape(H, d + dr)
        o = np.zeros((H, dv))
        seen = range(max(0, t - window + 1), t + 1)
        for hd in range(H):
            q_plain, q_rot = q[hd, :d], rotate(q[hd, d:], t, base, dims)
            sc = np.array([(q_plain @ (W[pre + "uk"][hd * d:(hd + 1) * d] @ lat[s]) + q_rot @ shared[s]) * mc["scale"] for s in seen])
            p = np.exp(sc - sc.max())
            p /= p.sum()
            o[hd] = sum(p[n] * (W[pre + "uv"][hd * dv:(hd + 1) * dv] @ lat[s]) for n, s in enumerate(seen))
        out[t] = o.reshape(-1)
    return out @ W[pre + "o"].T


MIXERS = {"wkv": wkv_mixer, "delta": delta_mixer, "latent_attention": latent_mixer}


def feed_forward(W, pre, h):
    a = W[pre + "act"]
    return xielu(h @ W[pre + "up"].T, a[0], a[1]) @ W[pre + "down"].T


def run(cfg, W, tokens, per_layer=None, window_override=None):
    """Logits [T, vocab] of a whole sequence.  window_override: {layer index: window} to state a WRONG model on purpose (sensitivity checks)."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)]
    for i, lc in enumerate(cfg["layers"]):
        p = "l%d." % i
        h = offset_norm(x, W[p + "norm1"], eps)
        h = h + time_conv(h, W[p + "canon1"])
        if lc["type"] == "latent_attention" and window_override and i in window_override:
            y = latent_mixer(W, p + "mix.", h, lc["mixer"], eps, window_override[i])
        else:
            y = MIXERS[lc["type"]](W, p + "mix.", h, lc["mixer"], eps)
        x = x + offset_norm(y, W[p + "norm1b"], eps)
        if lc.get("mlp"):
            h = offset_norm(x, W[p + "norm2"], eps)
            h = h + time_conv(h, W[p + "canon2"])
            x = x + offset_norm(feed_forward(W, p + "mlp.", h), W[p + "norm2b"], eps)
        if per_layer is not None:
            per_layer.append(x.copy())
    return offset_norm(x, W["final.norm"], eps) @ W["head"].T * cfg["logit_scale"]
