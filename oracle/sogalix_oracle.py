"""Plain, slow float64 implementation of the Sogalix layer-list design: test infrastructure only.

One function per mechanism, written from the equations, sharing nothing with the product path (libtlhip.so); numpy only.
Weights arrive as {checkpoint name: uint16 array of bf16 bits}; `config` is config.json's dictionary.

  norm        layer norm: (x - mean) / sqrt(var + eps) * w + b, var = mean of the squared deviations
  embedding   x = norm(embed[token])
  layer       x <- x + mixer(norm1(x));  x <- x + ff(norm2(x))  (a layer without feed-forward has the first half only)
  attention   q, k, v = W h with H query heads over G key/value heads;  q at position p times 1 + coef ln(floor((p + 1) / every) + 1);
              scores (q . k) scale over every j <= i;  weights exp(s_j) / (1 + sum_j exp(s_j)): a sink of score 0 that carries
              no value;  W_o
  latent      c_q = rms(W_dq h) w_dq, q = W_uq c_q, per head [dim plain | rot_dim rotated];  W_dkv h = [kv_rank | rot_dim]:
              c = rms(first part) w_dkv, the rest is ONE rotated key part for all heads;  keys of head n = [W_uk c | rotated part],
              values W_uv c;  rotary angles p f_i on interleaved pairs;  softmax over j <= i;  head n's output times
              sigmoid(W_g h)_n;  W_o.  A layer with kv_from = j reads layer j's (c, rotated part) instead of projecting its own.
  delta       r, k, v = W h per head;  decay w = exp(-e^-1/2 sigmoid(W_w2 tanh(W_w1 h) + w0)),  removal a = sigmoid(W_a h + b_a),
              u = k / sqrt(sum k^2 + 1e-6);  S <- diag(w) S - (a u)(u^T S) + k v^T (both terms read the old S);  o = S^T r;
              o / rms(o) per head, times the weight, times sigmoid(W_g h);  W_o
  ff          W_down act(W_up h), act(z) = sp(p) z^2 + z / 2 for z > 0, (1/2 + sp(q)) (e^z - 1 - z) + z / 2 otherwise
  output      norm, head
"""
import math

import numpy as np


def widen(bits):
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def rms(x, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def rotate(x, pos, dims, base):
    """x [T, ..., n]: the first `dims` of the last axis turn, (2i, 2i + 1) by pos * base^(-2i / dims)."""
    out = np.array(x, np.float64)
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    ang = np.asarray(pos, np.float64)[:, None] * f[None, :]
    ang = ang.reshape((ang.shape[0],) + (1,) * (x.ndim - 2) + (ang.shape[1],))
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * np.cos(ang) - v * np.sin(ang)
    out[..., 1:dims:2] = v * np.cos(ang) + u * np.sin(ang)
    return out


def query_temperature(pos, coef, every):
    return 1.0 + coef * np.log(np.floor((np.asarray(pos) + 1) / every) + 1.0)


def causal_attention(q, k, v, scale, q_pos, sink):
    """q [T, H, d], k [P, G, d], v [P, G, vd] (key j at position j) -> [T, H, vd]; sink: 1 joins the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        n = int(q_pos[t]) + 1
        for h in range(H):
            g = h // (H // G)
            s = (k[:n, g] @ q[t, h]) * scale
            m = max(s.max(), 0.0) if sink else s.max()
            e = np.exp(s - m)
            out[t, h] = (e @ v[:n, g]) / (e.sum() + (math.exp(-m) if sink else 0.0))
    return out


def generalized_delta(r, k, v, w, a, S):
    """One head: r, k, w, a [T, d], v [T, vd], S [d, vd] updated in place -> o [T, vd]."""
    o = np.zeros((r.shape[0], S.shape[1]))
    for t in range(r.shape[0]):
        u = k[t] / math.sqrt((k[t] * k[t]).sum() + 1e-6)
        old = S.copy()
        S[:] = w[t][:, None] * old - np.outer(a[t] * u, u @ old) + np.outer(k[t], v[t])
        o[t] = S.T @ r[t]
    return o


def xielu(z, p, q):
    neg = np.minimum(z, 0.0)
    return np.where(z > 0, softplus(p) * z * z + 0.5 * z, (0.5 + softplus(q)) * np.expm1(neg) - (0.5 + softplus(q)) * neg + 0.5 * z)


class SogalixOracle:
    def __init__(self, config, tensors):
        self.c = config
        self.w = {k: widen(v) for k, v in tensors.items()}
        self.eps = config["norm"]["eps"]
        self.reset()

    def reset(self):
        n = len(self.c["layers"])
        self.k = [None] * n      # attention: keys;  latent attention: the normalised latent c
        self.v = [None] * n      # attention: values;  latent attention: the rotated shared key part
        self.S = [None] * n      # delta rule: state [heads, dim, dim]
        self.pos = 0

    def norm(self, name, x):
        return layer_norm(x, self.w[name], self.w[name + ".b"], self.eps)

    def attention(self, i, h, pos):
        mx, p, w = self.c["layers"][i]["mixer"], f"l{i}.mix.", self.w
        T, H, G, d, vd = h.shape[0], mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        q = (h @ w[p + "q"].T).reshape(T, H, d)
        k = (h @ w[p + "k"].T).reshape(T, G, d)
        v = (h @ w[p + "v"].T).reshape(T, G, vd)
        qt = mx.get("q_temp")
        if qt:
            q = q * query_temperature(pos, qt["coef"], qt["every"])[:, None, None]
        self.k[i] = k if self.k[i] is None else np.concatenate([self.k[i], k])
        self.v[i] = v if self.v[i] is None else np.concatenate([self.v[i], v])
        o = causal_attention(q, self.k[i], self.v[i], mx["scale"], pos, sink=True)
        return o.reshape(T, -1) @ w[p + "o"].T

    def latent_attention(self, i, h, pos):
        mx, p, w = self.c["layers"][i]["mixer"], f"l{i}.mix.", self.w
        T, H, d, rd, vd, rank = h.shape[0], mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
        rot = mx["rot"]
        cq = rms(h @ w[p + "dq"].T, self.eps) * w[p + "dq.norm"]
        q = (cq @ w[p + "uq"].T).reshape(T, H, d + rd)
        q[..., d:] = rotate(q[..., d:], pos, rot["dims"], rot["base"])
        src = mx.get("kv_from")
        if src is None:
            ckv = h @ w[p + "dkv"].T
            c = rms(ckv[:, :rank], self.eps) * w[p + "dkv.norm"]
            kr = rotate(ckv[:, rank:], pos, rot["dims"], rot["base"])
            self.k[i] = c if self.k[i] is None else np.concatenate([self.k[i], c])
            self.v[i] = kr if self.v[i] is None else np.concatenate([self.v[i], kr])
            src = i
        c_all, kr_all = self.k[src], self.v[src]
        P = c_all.shape[0]
        kn = (c_all @ w[p + "uk"].T).reshape(P, H, d)
        keys = np.concatenate([kn, np.broadcast_to(kr_all[:, None, :], (P, H, rd))], axis=-1)
        vals = (c_all @ w[p + "uv"].T).reshape(P, H, vd)
        o = causal_attention(q, keys, vals, mx["scale"], pos, sink=False)
        o = o * sigmoid(h @ w[p + "g"].T)[:, :, None]
        return o.reshape(T, -1) @ w[p + "o"].T

    def general_delta(self, i, h):
        mx, p, w = self.c["layers"][i]["mixer"], f"l{i}.mix.", self.w
        T, H, d = h.shape[0], mx["heads"], mx["dim"]
        if self.S[i] is None:
            self.S[i] = np.zeros((H, d, d))
        r, k, v = ((h @ w[p + n].T).reshape(T, H, d) for n in "rkv")
        decay = np.exp(-math.exp(-0.5) * sigmoid(np.tanh(h @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).reshape(T, H, d)
        a = sigmoid(h @ w[p + "a"].T + w[p + "a.b"]).reshape(T, H, d)
        o = np.zeros((T, H, d))
        for n in range(H):
            o[:, n] = generalized_delta(r[:, n], k[:, n], v[:, n], decay[:, n], a[:, n], self.S[i][n])
        o = rms(o, self.eps).reshape(T, -1) * w[p + "norm"] * sigmoid(h @ w[p + "g"].T)
        return o @ w[p + "o"].T

    def ff(self, i, h):
        p, w = f"l{i}.mlp.", self.w
        if self.c["layers"][i]["mlp"]["kind"] != "dense":
            raise ValueError("unknown feed-forward kind")
        return xielu(h @ w[p + "up"].T, w[p + "act"][0], w[p + "act"][1]) @ w[p + "down"].T

    def forward(self, tokens, residuals=None):
        """The next tokens of the sequence: logits [T, vocab]. residuals: a list that receives x after every layer."""
        T = len(tokens)
        pos = np.arange(self.pos, self.pos + T)
        x = self.norm("embed.norm", self.w["embed"][np.asarray(tokens)])
        for i, L in enumerate(self.c["layers"]):
            h = self.norm(f"l{i}.norm1", x)
            if L["type"] == "attention":
                x = x + self.attention(i, h, pos)
            elif L["type"] == "latent_attention":
                x = x + self.latent_attention(i, h, pos)
            elif L["type"] == "general_delta":
                x = x + self.general_delta(i, h)
            else:
                raise ValueError(f"unknown layer type {L['type']!r}")
            if L.get("mlp") is not None:
                x = x + self.ff(i, self.norm(f"l{i}.norm2", x))
            if residuals is not None:
                residuals.append(x.copy())
        self.pos += T
        return self.norm("final.norm", x) @ self.w["head"].T

    def generate_greedy(self, prompt, n_new):
        """Arg-max continuation (first maximum), token by token after the prompt; resets the sequence first."""
        self.reset()
        logits = self.forward(list(prompt))[-1]
        out = []
        for _ in range(n_new):
            out.append(int(np.argmax(logits)))
            logits = self.forward([out[-1]])[0]
        return out
