"""Plain implementation of the Narurax decoder in float64, whole sequences only: one function a
mechanism, written from the equations, sharing no code with ``lockstep_amd``.  ``weights`` maps tensor
names to CPU tensors (any float dtype; integer tables as they are).

Notation: T tokens at positions 0 .. T-1, width W, H query heads, G key/value heads, key size d, value
size e.  All functions take and return float64."""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, times ``weight`` (None: no weight)."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z / (1.0 + torch.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def pair_embedding(tokens, table, pairs, mul_prev, mul_cur):
    """table[token] + pairs[(token before * mul_prev + token * mul_cur) mod B], B = rows of ``pairs`` - 1; the
    first token takes row B."""
    buckets = pairs.shape[0] - 1
    out = table[tokens].clone()
    for t in range(len(tokens)):
        row = buckets if t == 0 else (int(tokens[t - 1]) * mul_prev + int(tokens[t]) * mul_cur) % buckets
        out[t] = out[t] + pairs[row]
    return out


def shift_towards_previous(n, mu):
    """n[t] + (n[t-1] - n[t]) * mu, with zeros before the first row."""
    before = torch.cat([torch.zeros_like(n[:1]), n[:-1]])
    return n + (before - n) * mu


def frequencies(dims, base, scaling=None):
    """theta^(-2i/dims) for the pairs i = 0 .. dims/2 - 1; with ``scaling`` (factor, low, high, original) a
    frequency whose wavelength is below original/high stays, one above original/low is divided by factor,
    and between the two the share s = (original/wavelength - low) / (high - low) of the plain one is taken."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling is not None:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength > original / low:
                f = f / factor
            elif not wavelength < original / high:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate_neighbours(x, positions, freq):
    """x [T, heads, d]: dimensions (2i, 2i+1), i < len(freq), turn by the angle position * freq[i]."""
    out = x.clone()
    angle = positions.to(F64)[:, None] * freq[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    n = 2 * len(freq)
    a, b = x[..., 0:n:2], x[..., 1:n:2]
    out[..., 0:n:2] = a * c - b * s
    out[..., 1:n:2] = b * c + a * s
    return out


def visible(n, window, keep_first):
    """[n, n] bool: key j is seen from i iff j <= i and (i - j < window or j < keep_first)."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & ((i - j < window) | (j < keep_first))


def head_weights(q, k, scale, seen, sink):
    """Softmax weights [T, T] of one head whose denominator also holds exp(sink) (a number)."""
    s = (q @ k.T) * scale
    s = s.masked_fill(~seen, -math.inf)
    top = torch.clamp(s.max(dim=-1, keepdim=True).values, min=float(sink))
    e = torch.exp(s - top)
    return e / (e.sum(dim=-1, keepdim=True) + math.exp(float(sink)) * torch.exp(-top))


def short_convolution(x, taps):
    """x [T, C], taps [C, M]: y[t] = sum_m taps[:, m] x[t - (M-1) + m], zeros before the start."""
    n, m = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros((m - 1, x.shape[1]), dtype=x.dtype), x])
    return sum(padded[a:a + n] * taps[:, a] for a in range(m))


def delta_rule_with_channel_decay(q, k, v, beta, g):
    """One head.  q, k [T, d], v [T, e], beta [T], g [T, d] (a decay for every row of S):
    S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t."""
    n, d = q.shape
    S = torch.zeros((d, v.shape[1]), dtype=F64)
    out = torch.zeros((n, v.shape[1]), dtype=F64)
    for t in range(n):
        S = g[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def scored_experts(h, router, experts, top):
    """Scores sigmoid(router h); the ``top`` largest are chosen and each chosen expert reads score * h:
    sum over the chosen e of down_e(silu(gate_e x) * (up_e x)), x = score_e h."""
    scores = sigmoid(h @ router.T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = torch.topk(scores[t], top).indices.tolist()
        for e in chosen:
            gate, up, down = experts[e]
            x = scores[t, e] * h[t]
            out[t] = out[t] + down @ (silu(gate @ x) * (up @ x))
    return out


class PlainNarurax:
    def __init__(self, config: dict, weights: dict):
        self.c = config
        self.w = weights
        self.eps = float(config["norm"]["eps"])

    def t(self, name):
        value = self.w[name]
        return value.to(F64) if value.is_floating_point() else value

    def _window(self, m):
        return int(m["mask"]["size"]), int(m["mask"].get("keep_first", 0))

    def _rotated(self, m, q, k, positions):
        rot = m.get("rot")
        if not rot or not rot.get("dims"):
            return q, k
        f = frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        return rotate_neighbours(q, positions, f), rotate_neighbours(k, positions, f)

    def attention(self, i, m, h, positions):
        """v is k as it stood ahead of the rotation; a learned sink; weights mixed over the heads; a gate."""
        p = f"l{i}.mix"
        H, G, d = m["heads"], m["kv_heads"], m["dim"]
        n = h.shape[0]
        q = (h @ self.t(f"{p}.q").T).view(n, H, d)
        k = (h @ self.t(f"{p}.k").T).view(n, G, d)
        v = k.clone()
        q, k = self._rotated(m, q, k, positions)
        seen = visible(n, *self._window(m))
        sink = self.t(f"{p}.sink")
        w = torch.stack([head_weights(q[:, a], k[:, a // (H // G)], float(m["scale"]), seen, sink[a]) for a in range(H)])
        mixed = torch.einsum("ab,bij->aij", self.t(f"{p}.talk"), w)
        o = torch.stack([mixed[a] @ v[:, a // (H // G)] for a in range(H)], dim=1).reshape(n, -1)
        return (o * sigmoid(h @ self.t(f"{p}.g").T)) @ self.t(f"{p}.o").T

    def attention_2(self, i, m, h, positions):
        """Biases, a norm a head on q and k, stretched frequencies, a one in the softmax's denominator."""
        p = f"l{i}.mix"
        H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        n = h.shape[0]
        q = (h @ self.t(f"{p}.q").T + self.t(f"{p}.q.b")).view(n, H, d)
        k = (h @ self.t(f"{p}.k").T + self.t(f"{p}.k.b")).view(n, G, d)
        v = (h @ self.t(f"{p}.v").T + self.t(f"{p}.v.b")).view(n, G, e)
        q = rms_norm(q, self.t(f"{p}.q.norm"), self.eps)
        k = rms_norm(k, self.t(f"{p}.k.norm"), self.eps)
        q, k = self._rotated(m, q, k, positions)
        seen = visible(n, *self._window(m))
        o = torch.stack([head_weights(q[:, a], k[:, a // (H // G)], float(m["scale"]), seen, 0.0) @ v[:, a // (H // G)]
                         for a in range(H)], dim=1).reshape(n, -1)
        return o @ self.t(f"{p}.o").T + self.t(f"{p}.o.b")

    def channel_delta(self, i, m, h):
        p = f"l{i}.mix"
        H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        n = h.shape[0]
        q = silu(short_convolution(h @ self.t(f"{p}.q").T, self.t(f"{p}.q.conv"))).view(n, G, d)
        k = silu(short_convolution(h @ self.t(f"{p}.k").T, self.t(f"{p}.k.conv"))).view(n, G, d)
        v = silu(short_convolution(h @ self.t(f"{p}.v").T, self.t(f"{p}.v.conv"))).view(n, H, e)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = sigmoid(h @ self.t(f"{p}.b").T)
        logits = (h @ self.t(f"{p}.a1").T) @ self.t(f"{p}.a2").T + self.t(f"{p}.dt_bias")
        g = torch.exp(-torch.exp(self.t(f"{p}.A_log"))[None, :, None] * softplus(logits).view(n, H, d))
        o = torch.stack([delta_rule_with_channel_decay(q[:, a // (H // G)], k[:, a // (H // G)], v[:, a], beta[:, a], g[:, a])
                         for a in range(H)], dim=1)
        o = rms_norm(o, self.t(f"{p}.norm"), self.eps).reshape(n, -1)
        o = o * sigmoid((h @ self.t(f"{p}.g1").T) @ self.t(f"{p}.g2").T)
        return o @ self.t(f"{p}.o").T

    def mixer(self, i, layer, h, positions):
        m = layer["mixer"]
        if layer["type"] == "attention":
            return self.attention(i, m, h, positions)
        if layer["type"] == "attention_2":
            return self.attention_2(i, m, h, positions)
        if layer["type"] == "channel_delta":
            return self.channel_delta(i, m, h)
        raise ValueError(layer["type"])

    def feed_forward(self, i, mlp, h):
        p = f"l{i}.mlp"
        experts = [(self.t(f"{p}.e{e}.gate"), self.t(f"{p}.e{e}.up"), self.t(f"{p}.e{e}.down"))
                   for e in range(mlp["router"]["experts"])]
        return scored_experts(h, self.t(f"{p}.router"), experts, int(mlp["router"]["top"]))

    def forward(self, tokens, layers_out=None):
        """Logits [T, vocab] of a whole sequence; ``layers_out`` (a list) receives the residual stream after
        every layer."""
        tokens = torch.as_tensor(tokens, dtype=torch.int64)
        positions = torch.arange(len(tokens))
        pairs = self.c["embedding"]["bigram"]
        x = pair_embedding(tokens, self.t("embed"), self.t("bigram"), int(pairs["mul_prev"]), int(pairs["mul_cur"]))
        for i, layer in enumerate(self.c["layers"]):
            h = shift_towards_previous(rms_norm(x, self.t(f"l{i}.norm1"), self.eps), self.t(f"l{i}.shift"))
            x = x + self.mixer(i, layer, h, positions)
            if layer.get("mlp") is not None:
                x = x + self.feed_forward(i, layer["mlp"], rms_norm(x, self.t(f"l{i}.norm2"), self.eps))
            if layers_out is not None:
                layers_out.append(x.clone())
        return rms_norm(x, self.t("final.norm"), self.eps) @ self.t("head").T

    def generate_greedy(self, prompt, n_new):
        tokens = list(prompt)
        for _ in range(n_new):
            tokens.append(int(torch.argmax(self.forward(tokens)[-1])))
        return tokens[len(prompt):]
