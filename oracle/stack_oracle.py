"""Plain, slow float64 implementation of the Ralasun layer-list design: test infrastructure only.

One function per mechanism, written from the equations, sharing nothing with the product path (libtlhip.so); numpy only.
Weights arrive as {checkpoint name: uint16 array of bf16 bits}; `config` is config.json's dictionary.

  norm        y = x / sqrt(mean(x^2) + eps) * g          g = 1 + w for the block / embedding / final norms ("one_plus"),
                                                          g = w for the query and key norms
  layer       x <- x + norm1(mixer(x)),  x <- x + norm2(ff(x))      (the sublayers read x itself)
  mixer       q, k, v = W_q x, W_k x, W_v x;  q, k normalised over their WHOLE projection;  v mixed with the first mixing
              layer's v of the same token;  s_ij = scale * q_i . k_j for 0 <= i - j < window;  softmax;  W_o
  ff          router logits z = W_r x + b;  the `top` largest chosen, weights softmax over those;  expert(h) =
              W_down[min(W_gate h, L) * sigmoid(1.702 * min(W_gate h, L)) * (clip(W_up h, -L, L) + 1)];  + shared expert
"""
import numpy as np

ACT_ALPHA = 1.702


def widen(bits):
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def rms_norm(x, w, eps, one_plus):
    g = 1.0 + w if one_plus else w
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * g


def window_attention(q, k, v, heads, kv_heads, dim, vdim, window, scale, q_pos, k_pos):
    """q [Tq, heads*dim] at positions q_pos; k [Tk, kv_heads*dim], v [Tk, kv_heads*vdim] at positions k_pos."""
    Tq, Tk = q.shape[0], k.shape[0]
    q, k, v = q.reshape(Tq, heads, dim), k.reshape(Tk, kv_heads, dim), v.reshape(Tk, kv_heads, vdim)
    out = np.zeros((Tq, heads, vdim))
    rep = heads // kv_heads
    diff = np.asarray(q_pos)[:, None] - np.asarray(k_pos)[None, :]
    seen = diff >= 0
    if window and window > 0:
        seen &= diff < window
    for h in range(heads):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale
        s = np.where(seen, s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=1, keepdims=True)
        out[:, h] = p @ v[:, g]
    return out.reshape(Tq, heads * vdim)


def route(x, w_router, bias, top):
    """(ids [T, top] largest logit first, weights [T, top])."""
    z = x @ w_router.T + bias
    ids = np.argsort(-z, axis=1, kind="stable")[:, :top]
    zc = np.take_along_axis(z, ids, axis=1)
    e = np.exp(zc - zc.max(axis=1, keepdims=True))
    return ids, e / e.sum(axis=1, keepdims=True)


def clamped_glu(h, w_gate, w_up, w_down, limit):
    g = np.minimum(h @ w_gate.T, limit)
    u = np.clip(h @ w_up.T, -limit, limit)
    return (g / (1.0 + np.exp(-ACT_ALPHA * g)) * (u + 1.0)) @ w_down.T


class StackOracle:
    def __init__(self, config, tensors):
        self.c = config
        self.w = {k: widen(v) for k, v in tensors.items()}
        self.eps = config["norm"]["eps"]
        self.reset()

    def reset(self):
        n = len(self.c["layers"])
        self.k = [None] * n
        self.v = [None] * n
        self.pos = 0

    def moe(self, i, x):
        ml, p, w = self.c["layers"][i]["mlp"], f"l{i}.mlp.", self.w
        ids, wts = route(x, w[p + "router"], w[p + "router.b"], ml["router"]["top"])
        y = np.zeros_like(x)
        for t in range(x.shape[0]):
            for e, a in zip(ids[t], wts[t]):
                q = p + f"e{e}."
                y[t] += a * clamped_glu(x[t], w[q + "gate"], w[q + "up"], w[q + "down"], ml["expert"]["limit"])
        if ml.get("shared"):
            q = p + "shared."
            y += clamped_glu(x, w[q + "gate"], w[q + "up"], w[q + "down"], ml["shared"]["limit"])
        return y

    def forward(self, tokens, layers_out=None):
        """Feeds `tokens` at the positions after what was fed before (the caches persist); returns logits [T, vocab]."""
        w, c = self.w, self.c
        T = len(tokens)
        q_pos = np.arange(self.pos, self.pos + T)
        x = rms_norm(w["embed"][np.asarray(tokens)], w["embed.norm"], self.eps, True)
        v_first = None
        for i, L in enumerate(c["layers"]):
            mx, p = L["mixer"], f"l{i}.mix."
            q = rms_norm(x @ w[p + "q"].T, w[p + "q.norm"], self.eps, False)
            k = rms_norm(x @ w[p + "k"].T, w[p + "k.norm"], self.eps, False)
            v = x @ w[p + "v"].T
            if mx.get("v_mix"):
                if v_first is None:
                    v_first = v
                else:
                    lam = float(np.asarray(w[p + "vmix"]).reshape(-1)[0])
                    v = (1.0 - lam) * v + lam * v_first
            self.k[i] = k if self.k[i] is None else np.concatenate([self.k[i], k])
            self.v[i] = v if self.v[i] is None else np.concatenate([self.v[i], v])
            window = (mx.get("mask") or {}).get("size", 0)
            a = window_attention(q, self.k[i], self.v[i], mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"], window,
                                 mx["scale"], q_pos, np.arange(self.pos + T))
            x = x + rms_norm(a @ w[p + "o"].T, w[f"l{i}.norm1"], self.eps, True)
            if L.get("mlp") is not None:
                x = x + rms_norm(self.moe(i, x), w[f"l{i}.norm2"], self.eps, True)
            if layers_out is not None:
                layers_out.append(x.copy())
        self.pos += T
        return rms_norm(x, w["final.norm"], self.eps, True) @ w["head"].T

    def generate_greedy(self, prompt, n):
        self.reset()
        logits = self.forward(prompt)
        out = [int(np.argmax(logits[-1]))]
        while len(out) < n:
            out.append(int(np.argmax(self.forward([out[-1]])[-1])))
        return out
