"""Plain, slow float64 implementation of the Potipel layer-list design: test infrastructure only.

One function per mechanism, written from the equations, sharing nothing with the product path (libtlhip.so); numpy only.
Weights arrive as {checkpoint name: uint16 array of bf16 bits}; `config` is config.json's dictionary.

  norm        RMS norm with plain weights: x / sqrt(mean(x^2) + eps) * w
  embedding   x = embed[token] * embedding.scale
  layer       x <- x + mixer(C1(norm1(x)));  x <- x + ff(C2(norm2(x)));  C(h)_t = h_t + sum_j c[:, j] h_(t - taps + 1 + j): a causal
              convolution over time per channel added to its own input (zeros before the sequence); a layer may use an earlier
              layer's tensors (weights_of) with a state of its own
  attention   two score maps per head (q, k rows laid out head by head as [map 1 | map 2]) over the same values; q and k
              RMS-normed per head and map with one weight of size dim each; causal softmax of (q . k) scale per map;
              o = a1 - lambda a2, lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff; o / rms(o) (1 - diff); times sigmoid(W_g h); W_o
  hgrn2       q = silu(W_q h), f = l + (1 - l) sigmoid(W_f h + b); S <- diag(f) S + (1 - f) v^T; o = S^T q; RMS norm per head; W_o
  parallel    left_scale left + right_scale right, both reading the same input:
              left   q, k, v = W h + b, a causal convolution over time on each (no activation); score = cap tanh((q . k) scale / cap)
                     - r1 ln(1 + r2 (i - j)); window 0 <= i - j < size; softmax whose denominator also holds exp(sink_head); W_o
              right  q, k (kv_heads), v (heads) through a causal convolution and silu; q, k unit vectors (1e-6), q dim^-1/2;
                     beta = sigmoid(W_b h); g = exp(-exp(A_log) softplus(W_a h + dt_bias)) per head;
                     S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q; o / rms(o) w silu(W_g h); W_o
  ff          dense: W_down (relu(W_gate h) (W_up h));  experts: s = sigmoid(W_router h), choice = s + correction, groups of
              neighbours scored by their two best choices, the best `keep` groups stay, the `top` best choices among them are
              taken, weights = s of the taken (not normalised); expert: g = min(W_gate h, L), u = clip(W_up h, -L, L),
              W_down (g sigmoid(1.702 g) (u + 1))
  output      norm, head
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


def rms(x, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def causal_conv(u, w, hist):
    """u [T, C] inputs, w [C, taps] (the last column is the current token's), hist [taps - 1, C] the inputs before u (oldest
    first) -> (y [T, C], the new history)."""
    taps = w.shape[1]
    full = np.concatenate([hist, u]) if taps > 1 else u
    y = np.zeros_like(u)
    for j in range(taps):
        y += full[j:j + u.shape[0]] * w[:, j]
    return y, (full[full.shape[0] - (taps - 1):] if taps > 1 else hist)


def softmax_attention(q, k, v, scale, q_pos, window=0, softcap=0.0, r1=None, r2=None, sink=None):
    """q [T, H, d] at positions q_pos, k [P, G, d], v [P, G, vd] (key j at position j) -> [T, H, vd].
    window > 0: only 0 <= i - j < window; softcap > 0: s <- cap tanh(s / cap); r1, r2 [H]: s <- s - r1 ln(1 + r2 (i - j));
    sink [H]: exp(sink) joins the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        i = int(q_pos[t])
        lo = max(0, i - window + 1) if window > 0 else 0
        dist = i - np.arange(lo, i + 1)
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:i + 1, g] @ q[t, h]) * scale
            if softcap > 0:
                s = softcap * np.tanh(s / softcap)
            if r1 is not None:
                s = s - r1[h] * np.log1p(r2[h] * dist)
            m = s.max() if sink is None else max(s.max(), sink[h])
            e = np.exp(s - m)
            out[t, h] = (e @ v[lo:i + 1, g]) / (e.sum() + (0.0 if sink is None else math.exp(sink[h] - m)))
    return out


def differential_combine(a1, a2, lam, diff, eps):
    """a1, a2 [T, H, vd] -> (a1 - lam a2) / rms (1 - diff)."""
    return rms(a1 - lam * a2, eps) * (1.0 - diff)


def gated_linear_recurrence(q, f, v, S):
    """One head: q, f [T, d], v [T, vd], S [d, vd] updated in place: S <- diag(f) S + (1 - f) v^T; o = S^T q."""
    o = np.zeros((q.shape[0], S.shape[1]))
    for t in range(q.shape[0]):
        S[:] = f[t][:, None] * S + np.outer(1.0 - f[t], v[t])
        o[t] = S.T @ q[t]
    return o


def gated_delta_rule(q, k, v, beta, g, S):
    """One head: q, k [T, d], v [T, vd], beta, g [T], S [d, vd] updated in place."""
    o = np.zeros((q.shape[0], S.shape[1]))
    for t in range(q.shape[0]):
        S *= g[t]
        u = beta[t] * (v[t] - S.T @ k[t])
        S += np.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o


def route_sigmoid_groups(z, correction, top, groups, keep):
    """z [E] router logits -> (ids [top] best choice first, weights [top])."""
    s = sigmoid(z)
    choice = s + correction
    E = z.shape[0]
    per = E // groups
    score = np.array([np.sort(choice[g * per:(g + 1) * per])[::-1][:2].sum() for g in range(groups)])
    kept = np.argsort(-score, kind="stable")[:keep]
    masked = np.full(E, -np.inf)
    for g in kept:
        masked[g * per:(g + 1) * per] = choice[g * per:(g + 1) * per]
    ids = np.argsort(-masked, kind="stable")[:top]
    return ids, s[ids]


def clamped_expert(h, gate, up, down, limit):
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


class PotipelOracle:
    def __init__(self, config, tensors):
        self.c = config
        self.w = {k: widen(v) for k, v in tensors.items()}
        self.eps = config["norm"]["eps"]
        self.taps = config["canon"]["taps"]
        self.reset()

    def reset(self):
        self.state = [dict() for _ in self.c["layers"]]
        self.pos = 0

    def owner(self, i):
        while "weights_of" in self.c["layers"][i]:
            i = self.c["layers"][i]["weights_of"]
        return i

    def norm(self, name, x):
        return rms(x, self.eps) * self.w[name]

    def canon(self, i, which, h):
        key = "canon%d" % which
        w = self.w[f"l{self.owner(i)}.{key}"]
        hist = self.state[i].get(key)
        if hist is None:
            hist = np.zeros((self.taps - 1, h.shape[1]))
        y, self.state[i][key] = causal_conv(h, w, hist)
        return h + y

    def conv(self, i, name, u, act=None):
        """The short convolution '<name>.conv' of layer i on the projected values u, with its state."""
        w = self.w[name + ".conv"]
        hist = self.state[i].get(name)
        if hist is None:
            hist = np.zeros((w.shape[1] - 1, u.shape[1]))
        y, self.state[i][name] = causal_conv(u, w, hist)
        return act(y) if act else y

    def append(self, i, key, rows):
        old = self.state[i].get(key)
        self.state[i][key] = rows if old is None else np.concatenate([old, rows])
        return self.state[i][key]

    def attention(self, i, h, pos):
        mx, p, w = self.c["layers"][i]["mixer"], f"l{self.owner(i)}.mix.", self.w
        T, H, G, d, vd = h.shape[0], mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        q = rms((h @ w[p + "q"].T).reshape(T, H, 2, d), self.eps) * w[p + "q.norm"]
        k = rms((h @ w[p + "k"].T).reshape(T, G, 2, d), self.eps) * w[p + "k.norm"]
        v = (h @ w[p + "v"].T).reshape(T, G, vd)
        k = self.append(i, "k", k)
        v = self.append(i, "v", v)
        a = [softmax_attention(q[:, :, m], k[:, :, m], v, mx["scale"], pos) for m in range(2)]
        lam = math.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - math.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + mx["diff"]
        o = differential_combine(a[0], a[1], lam, mx["diff"], self.eps).reshape(T, -1)
        return (o * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T

    def hgrn2(self, i, h):
        mx, p, w = self.c["layers"][i]["mixer"], f"l{self.owner(i)}.mix.", self.w
        T, H, d, vd = h.shape[0], mx["heads"], mx["dim"], mx["vdim"]
        q = silu(h @ w[p + "q"].T).reshape(T, H, d)
        v = (h @ w[p + "v"].T).reshape(T, H, vd)
        low = w[p + "lower"]
        f = (low + (1.0 - low) * sigmoid(h @ w[p + "f"].T + w[p + "f.b"])).reshape(T, H, d)
        S = self.state[i].setdefault("S", np.zeros((H, d, vd)))
        o = np.stack([gated_linear_recurrence(q[:, n], f[:, n], v[:, n], S[n]) for n in range(H)], axis=1)
        return (rms(o, self.eps) * w[p + "norm"]).reshape(T, -1) @ w[p + "o"].T

    def window_attention(self, i, h, pos):
        mx, p, w = self.c["layers"][i]["mixer"]["left"], f"l{self.owner(i)}.mix.left.", self.w
        T, H, G, d, vd = h.shape[0], mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        q, k, v = (self.conv(i, p + n, h @ w[p + n].T + w[p + n + ".b"]) for n in "qkv")
        k = self.append(i, "k", k.reshape(T, G, d))
        v = self.append(i, "v", v.reshape(T, G, vd))
        o = softmax_attention(q.reshape(T, H, d), k, v, mx["scale"], pos, window=(mx.get("mask") or {}).get("size", 0),
                              softcap=mx.get("softcap") or 0.0, r1=w[p + "r1"], r2=w[p + "r2"], sink=w[p + "sink"])
        return o.reshape(T, -1) @ w[p + "o"].T

    def delta_rule(self, i, h):
        mx, p, w = self.c["layers"][i]["mixer"]["right"], f"l{self.owner(i)}.mix.right.", self.w
        T, H, G, d, vd = h.shape[0], mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        q, k, v = (self.conv(i, p + n, h @ w[p + n].T, silu) for n in "qkv")
        q = q.reshape(T, G, d)
        k = k.reshape(T, G, d)
        q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
        k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
        v = v.reshape(T, H, vd)
        beta = sigmoid(h @ w[p + "b"].T)
        g = np.exp(-np.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
        S = self.state[i].setdefault("S", np.zeros((H, d, vd)))
        o = np.stack([gated_delta_rule(q[:, n // (H // G)], k[:, n // (H // G)], v[:, n], beta[:, n], g[:, n], S[n])
                      for n in range(H)], axis=1)
        o = (rms(o, self.eps) * w[p + "norm"]).reshape(T, -1) * silu(h @ w[p + "g"].T)
        return o @ w[p + "o"].T

    def route(self, i, h):
        """ids, weights [T, top] of layer i's router."""
        r, p = self.c["layers"][i]["mlp"]["router"], f"l{self.owner(i)}.mlp."
        z = h @ self.w[p + "router"].T
        picks = [route_sigmoid_groups(z[t], self.w[p + "correction"], r["top"], r["groups"]["count"], r["groups"]["keep"])
                 for t in range(h.shape[0])]
        return np.array([a for a, _ in picks]), np.array([b for _, b in picks])

    def ff(self, i, h):
        m, p, w = self.c["layers"][i]["mlp"], f"l{self.owner(i)}.mlp.", self.w
        if m["kind"] == "dense":
            return (np.maximum(h @ w[p + "gate"].T, 0.0) * (h @ w[p + "up"].T)) @ w[p + "down"].T
        if m["kind"] != "moe":
            raise ValueError("unknown feed-forward kind")
        ids, wts = self.route(i, h)
        out = np.zeros_like(h)
        for t in range(h.shape[0]):
            for e, a in zip(ids[t], wts[t]):
                q = f"{p}e{e}."
                out[t] += a * clamped_expert(h[t], w[q + "gate"], w[q + "up"], w[q + "down"], m["expert"]["limit"])
        return out

    def forward(self, tokens, residuals=None):
        """The next tokens of the sequence: logits [T, vocab]. residuals: a list that receives x after every layer."""
        T = len(tokens)
        pos = np.arange(self.pos, self.pos + T)
        x = self.w["embed"][np.asarray(tokens)] * self.c["embedding"]["scale"]
        for i, L in enumerate(self.c["layers"]):
            o = self.owner(i)
            h = self.canon(i, 1, self.norm(f"l{o}.norm1", x))
            if L["type"] == "attention":
                x = x + self.attention(i, h, pos)
            elif L["type"] == "hgrn2":
                x = x + self.hgrn2(i, h)
            elif L["type"] == "parallel":
                x = x + L["mixer"]["left_scale"] * self.window_attention(i, h, pos) + L["mixer"]["right_scale"] * self.delta_rule(i, h)
            else:
                raise ValueError(f"unknown layer type {L['type']!r}")
            if L.get("mlp") is not None:
                x = x + self.ff(i, self.canon(i, 2, self.norm(f"l{o}.norm2", x)))
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
