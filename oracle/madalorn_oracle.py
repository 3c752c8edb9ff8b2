"""Plain, slow float64 implementation of the Madalorn layer-list design: test infrastructure only.

One function per mechanism, written from the equations, sharing nothing with the product path (libtlhip.so); numpy only.
Weights arrive as {checkpoint name: uint16 array of bf16 bits}; `config` is config.json's dictionary.

  norm        Dynamic Tanh: y = tanh(alpha x) * w + b (no mean, no variance)
  layer       h = norm1(x);  x <- x + mixer(h) + ff(h)            (one norm, both sublayers read its output)
  attention   q = W_q h, k = W_k h, the values are the keys as projected;  rotary angles p * f_i on interleaved pairs of the
              first rot.dims dimensions with the blended frequencies of a context extension;  q, k divided by their root mean
              square per head;  position i sees j <= i with i - j < size or j < keep_first;  weight = sigmoid(scale q.k + pb_h),
              not normalised over the keys;  W_o
  delta       q, k, v projections -> short causal convolution per channel -> silu;  q, k unit vectors per head (q also times
              dim^-1/2);  beta = sigmoid(W_b h);  decay g = exp(-exp(A_log) softplus(W_a2 W_a1 h + dt_bias)) per head and key
              channel;  S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;  o / rms(o) * w * sigmoid(W_g2 W_g1 h);  W_o
  ff          dense: W_down[silu(W_gate h) * W_up h];  experts: scores = softmax(W_r h) over all experts, groups of
              neighbours ranked by their best score, the `top` best experts of the kept groups, weights = their scores
              divided by their sum;  + sigmoid(w_sg . h) * shared expert
  output      final norm, head, cap * tanh(logits / cap)
"""
import math

import numpy as np


def widen(bits):
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def dyt(x, alpha, w, b):
    return np.tanh(alpha * x) * w + b


def rotary_frequencies(rot):
    """f_i for i < dims / 2 and the factor on cos and sin."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = sc["factor"], sc["original"]

    def turn_dim(t):
        return dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(sc["fast"])), 0)
    hi = min(math.ceil(turn_dim(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, pos, rot):
    """x [T, heads, dim] at positions pos [T]; interleaved pairs (2i, 2i + 1) of the first rot.dims dimensions."""
    if not rot:
        return x.copy()
    f, m = rotary_frequencies(rot)
    n = rot["dims"]
    a = np.asarray(pos, np.float64)[:, None, None] * f[None, None, :]
    c, s = np.cos(a) * m, np.sin(a) * m
    out = x.copy()
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid_window_attention(q, k, v, pb, scale, size, keep_first, q_pos, k_pos):
    """q [Tq, H, dim], k [Tk, G, dim], v [Tk, G, vdim]; returns [Tq, H, vdim]."""
    Tq, H, _ = q.shape
    G = k.shape[1]
    qp, kp = np.asarray(q_pos)[:, None], np.asarray(k_pos)[None, :]
    seen = (kp <= qp) & ((qp - kp < size) | (kp < keep_first))
    out = np.zeros((Tq, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        w = np.where(seen, sigmoid((q[:, h] @ k[:, g].T) * scale + pb[h]), 0.0)
        out[:, h] = w @ v[:, g]
    return out


def short_conv(x, w, history):
    """x [T, C], w [C, taps] (last column = current token), history [taps - 1, C] (zeros at the start of a sequence).
    Returns (y [T, C], new history)."""
    taps = w.shape[1]
    ext = np.concatenate([history, x], axis=0)
    y = np.zeros_like(x)
    for j in range(taps):
        y += ext[j:j + x.shape[0]] * w[:, j][None, :]
    return y, ext[ext.shape[0] - (taps - 1):]


def delta_rule(q, k, v, beta, g, S):
    """One head, token by token. q, k, g [T, dim]; v [T, vdim]; beta [T]; S [dim, vdim] (updated in place). Returns o [T, vdim]."""
    o = np.zeros_like(v)
    for t in range(q.shape[0]):
        S *= g[t][:, None]
        u = beta[t] * (v[t] - S.T @ k[t])
        S += np.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o


def route_groups(h, w_router, top, count, keep):
    """(ids [T, top], weights [T, top]): softmax over all experts, the best `keep` of `count` groups, top experts of those."""
    z = h @ w_router.T
    z = z - z.max(axis=1, keepdims=True)
    s = np.exp(z)
    s /= s.sum(axis=1, keepdims=True)
    T, E = s.shape
    per = E // count
    gs = s.reshape(T, count, per).max(axis=2)
    kept = np.argsort(-gs, axis=1, kind="stable")[:, :keep]
    allowed = np.zeros((T, count), bool)
    np.put_along_axis(allowed, kept, True, axis=1)
    masked = np.where(np.repeat(allowed, per, axis=1), s, -1.0)
    ids = np.argsort(-masked, axis=1, kind="stable")[:, :top]
    w = np.take_along_axis(s, ids, axis=1)
    return ids, w / (w.sum(axis=1, keepdims=True) + 1e-20)


def silu_glu(h, w_gate, w_up, w_down):
    return (silu(h @ w_gate.T) * (h @ w_up.T)) @ w_down.T


class MadalornOracle:
    def __init__(self, config, tensors):
        self.c = config
        self.w = {k: widen(v) for k, v in tensors.items()}
        self.eps = config["norm"]["eps"]
        self.reset()

    def reset(self):
        n = len(self.c["layers"])
        self.k = [None] * n      # rotated, normalised keys per attention layer
        self.v = [None] * n      # values (the keys as projected)
        self.S = [None] * n      # delta state [heads, dim, vdim]
        self.hist = [None] * n   # convolution inputs of the last taps - 1 tokens: (q, k, v)
        self.pos = 0

    def src(self, i):
        while "weights_of" in self.c["layers"][i]:
            i = self.c["layers"][i]["weights_of"]
        return i

    def norm(self, name, x):
        return dyt(x, self.w[name + ".alpha"].reshape(()), self.w[name], self.w[name + ".b"])

    def attention(self, i, h, pos):
        mx, p, w = self.c["layers"][i]["mixer"], f"l{self.src(i)}.mix.", self.w
        T, H, G, d = h.shape[0], mx["heads"], mx["kv_heads"], mx["dim"]
        q = (h @ w[p + "q"].T).reshape(T, H, d)
        k = (h @ w[p + "k"].T).reshape(T, G, d)
        v = k.copy()
        q = unit_rms(rotate(q, pos, mx.get("rot")), self.eps)
        k = unit_rms(rotate(k, pos, mx.get("rot")), self.eps)
        self.k[i] = k if self.k[i] is None else np.concatenate([self.k[i], k])
        self.v[i] = v if self.v[i] is None else np.concatenate([self.v[i], v])
        mask = mx.get("mask") or {}
        o = sigmoid_window_attention(q, self.k[i], self.v[i], w[p + "pb"], mx["scale"], mask.get("size", 1 << 60),
                                     mask.get("keep_first", 0), pos, np.arange(self.k[i].shape[0]))
        return o.reshape(T, -1) @ w[p + "o"].T

    def channel_delta(self, i, h):
        mx, p, w = self.c["layers"][i]["mixer"], f"l{self.src(i)}.mix.", self.w
        T, H, G, d, vd, taps = h.shape[0], mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"], mx["conv"]
        if self.S[i] is None:
            self.S[i] = np.zeros((H, d, vd))
            self.hist[i] = [np.zeros((taps - 1, G * d)), np.zeros((taps - 1, G * d)), np.zeros((taps - 1, H * vd))]
        outs = []
        for j, n in enumerate("qkv"):
            y, self.hist[i][j] = short_conv(h @ w[p + n].T, w[p + n + ".conv"], self.hist[i][j])
            outs.append(silu(y))
        q, k, v = outs[0].reshape(T, G, d), outs[1].reshape(T, G, d), outs[2].reshape(T, H, vd)
        q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
        k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
        beta = sigmoid(h @ w[p + "b"].T)
        dt = softplus((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).reshape(T, H, d)
        g = np.exp(-np.exp(w[p + "A_log"])[None, :, None] * dt)
        o = np.zeros((T, H, vd))
        for hh in range(H):
            kv = hh // (H // G)
            o[:, hh] = delta_rule(q[:, kv], k[:, kv], v[:, hh], beta[:, hh], g[:, hh], self.S[i][hh])
        gate = sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).reshape(T, H, vd)
        o = unit_rms(o, self.eps) * w[p + "norm"] * gate
        return o.reshape(T, -1) @ w[p + "o"].T

    def ff(self, i, h):
        ml, p, w = self.c["layers"][i]["mlp"], f"l{self.src(i)}.mlp.", self.w
        if ml is None:
            return np.zeros_like(h)
        if ml["kind"] == "dense":
            return silu_glu(h, w[p + "gate"], w[p + "up"], w[p + "down"])
        r = ml["router"]
        groups = r.get("groups") or {"count": 1, "keep": 1}
        ids, wts = route_groups(h, w[p + "router"], r["top"], groups["count"], groups["keep"])
        y = np.zeros_like(h)
        for t in range(h.shape[0]):
            for j in range(ids.shape[1]):
                e = f"{p}e{ids[t, j]}."
                y[t] += wts[t, j] * silu_glu(h[t:t + 1], w[e + "gate"], w[e + "up"], w[e + "down"])[0]
        if ml.get("shared"):
            s = p + "shared."
            y += sigmoid(h @ w[s + "sg"].T) * silu_glu(h, w[s + "gate"], w[s + "up"], w[s + "down"])
        return y

    def forward(self, tokens, residuals=None):
        """The next tokens of the sequence: logits [T, vocab]. residuals: a list that receives x after every layer."""
        T = len(tokens)
        pos = np.arange(self.pos, self.pos + T)
        x = self.w["embed"][np.asarray(tokens)]
        for i, L in enumerate(self.c["layers"]):
            h = self.norm(f"l{self.src(i)}.norm1", x)
            m = self.attention(i, h, pos) if L["type"] == "attention" else self.channel_delta(i, h)
            x = x + (m + self.ff(i, h))
            if residuals is not None:
                residuals.append(x.copy())
        self.pos += T
        z = self.norm("final.norm", x) @ self.w["head"].T
        cap = self.c.get("logit_softcap")
        return cap * np.tanh(z / cap) if cap else z

    def generate_greedy(self, prompt, n_new):
        """Arg-max continuation (first maximum), token by token after the prompt; resets the sequence first."""
        self.reset()
        logits = self.forward(list(prompt))[-1]
        out = []
        for _ in range(n_new):
            out.append(int(np.argmax(logits)))
            logits = self.forward([out[-1]])[0]
        return out
