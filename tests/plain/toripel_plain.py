"""A plain, slow implementation of the Toripel decoder in float64 on the CPU: one function per
mechanism, written from the equations, sharing no code with the engine.  It reads the same
``config.json`` dictionary and the same tensor names as the engine and runs whole sequences
only (no cache, no portions): what the engine must reproduce however it cuts the work.

Notation: ``h`` a sublayer's normalised input ``[T, width]``; positions count from 0; ``i`` is the
position of a query and ``j`` of a key; ``X [T, n, width]`` the n residual streams."""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def centred_norm(x, weight, eps):
    """A root-mean-square norm whose weight is stored as its distance from one."""
    return rms(x, eps) * (1.0 + weight)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def in_window(n, size):
    """visible[i, j]: 0 <= i - j < size (every j <= i when ``size`` is None)."""
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    seen = j <= i
    return seen if size is None else seen & (i - j < size)


def softmax_attention(q, k, v, scale, visible, sink=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads kv head h // (H/G).  The weights of a
    row are exp(s_j) over the sum of exp(s) of its visible keys, plus exp(sink_h) where a sink [H] is
    given: a term of the denominator with no key and no value."""
    n, heads, _ = q.shape
    group = heads // k.shape[1]
    out = torch.zeros((n, heads, v.shape[2]), dtype=F64)
    for h in range(heads):
        s = (q[:, h] @ k[:, h // group].T) * scale
        s = s.masked_fill(~visible, float("-inf"))
        top = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[h].reshape(1, 1))
        e = torch.exp(s - top)
        total = e.sum(dim=-1, keepdim=True)
        if sink is not None:
            total = total + torch.exp(sink[h] - top)
        out[:, h] = (e / total) @ v[:, h // group]
    return out


def stretched_frequencies(dims, base, scaling=None):
    """(f [dims/2], magnitude).  f_i = base^(-2i/dims).  With ``scaling`` (factor, original, fast, slow):
    the pair index at which a rotation makes t turns within ``original`` positions is
    c(t) = dims ln(original / (2 pi t)) / (2 ln base); pairs below floor(c(fast)) keep their frequency,
    pairs above ceil(c(slow)) have it divided by ``factor``, pairs between are blended linearly in the
    index; cosines and sines are multiplied by 0.1 ln(factor) + 1."""
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return torch.tensor(f, dtype=F64), 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turns_at(t):
        return dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turns_at(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turns_at(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(1.0, max(0.0, (i - lo) / max(hi - lo, 0.001)))
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, frequencies, magnitude=1.0):
    """The first 2 len(frequencies) dimensions of the last axis of ``x [T, ..., d]`` in neighbouring pairs:
    (u, v) at position p becomes (u c - v s, v c + u s), c = magnitude cos(p f_i), s = magnitude sin(p f_i)."""
    dims = 2 * len(frequencies)
    angle = positions.to(F64)[:, None] * frequencies[None, :]
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (dims // 2,)
    c, s = (angle.cos() * magnitude).reshape(shape), (angle.sin() * magnitude).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def short_convolution(x, taps):
    """y[t, c] = sum_m taps[c, m] x[t - (M - 1) + m, c] with zeros before the start: the last column
    of ``taps [C, M]`` multiplies the current token."""
    n, m = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros((m - 1, x.shape[1]), dtype=F64), x])
    y = torch.zeros_like(x)
    for a in range(m):
        y = y + padded[a:a + n] * taps[:, a]
    return y


def gated_delta_rule(q, k, v, beta, decay):
    """Per head, over time, with S [d, dv] zero at the start:
    S <- decay_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t.
    q, k [T, H, d]; v [T, H, dv]; beta, decay [T, H]."""
    n, heads, d = q.shape
    dv = v.shape[2]
    out = torch.zeros((n, heads, dv), dtype=F64)
    for h in range(heads):
        state = torch.zeros((d, dv), dtype=F64)
        for t in range(n):
            state = decay[t, h] * state
            u = beta[t, h] * (v[t, h] - state.T @ k[t, h])
            state = state + torch.outer(k[t, h], u)
            out[t, h] = state.T @ q[t, h]
    return out


def tabled_experts(h, tokens, table, experts):
    """Every token runs the experts its id's row of ``table [vocab, top]`` names, each weighing 1/top.
    ``experts``: a list of (gate, up, down) matrices; an expert is down(silu(gate h) * (up h))."""
    out = torch.zeros_like(h)
    top = table.shape[1]
    for t in range(h.shape[0]):
        for e in table[int(tokens[t])].tolist():
            gate, up, down = experts[e]
            out[t] += (down @ (silu(gate @ h[t]) * (up @ h[t]))) / top
    return out


def read_streams(X, weights_in):
    """u = sum_s in[s] X_s."""
    return torch.einsum("s,tsw->tw", weights_in, X)


def write_streams(X, y, mix, weights_out):
    """X'_t = sum_s mix[s, t] X_s + out[t] y, all streams at once from the old ones."""
    return torch.einsum("sr,tsw->trw", mix, X) + weights_out[None, :, None] * y[:, None, :]


class PlainToripel:
    def __init__(self, config: dict, weights: dict):
        self.c = config
        self.w = {name: t.to(F64) if t.is_floating_point() else t.to(torch.int64) for name, t in weights.items()}
        self.eps = float(config["norm"]["eps"])
        self.streams = config.get("streams")

    def t(self, name):
        return self.w[name]

    # -- mixers -----------------------------------------------------------------------------
    def attention(self, i, m, h, positions):
        p = f"l{i}.mix"
        n = h.shape[0]
        heads, groups, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        q = (h @ self.t(f"{p}.q").T + self.t(f"{p}.q.b")).reshape(n, heads, d)
        k = (h @ self.t(f"{p}.k").T + self.t(f"{p}.k.b")).reshape(n, groups, d)
        v = (h @ self.t(f"{p}.v").T + self.t(f"{p}.v.b")).reshape(n, groups, dv)
        q, k = rms(q, self.eps), rms(k, self.eps)
        size = m["mask"]["size"] if m.get("mask") else None
        o = softmax_attention(q, k, v, float(m["scale"]), in_window(n, size))
        return o.reshape(n, heads * dv) @ self.t(f"{p}.o").T

    def latent(self, i, m, h, positions):
        """(latent c [T, kv_rank], rotated shared key part [T, rot_dim]) of layer i."""
        p = f"l{i}.mix"
        rank, rot = m["kv_rank"], m["rot_dim"]
        down = h @ self.t(f"{p}.dkv").T
        c = rms(down[:, :rank], self.eps) * self.t(f"{p}.dkv.norm")
        f, magnitude = stretched_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
        return c, rotate_pairs(down[:, rank:rank + rot], positions, f, magnitude)

    def latent_attention(self, i, m, h, positions, kept):
        p = f"l{i}.mix"
        n = h.shape[0]
        heads, d, rot, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        cq = rms(h @ self.t(f"{p}.dq").T, self.eps) * self.t(f"{p}.dq.norm")
        q = (cq @ self.t(f"{p}.uq").T).reshape(n, heads, d + rot)
        f, magnitude = stretched_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
        q_rot = rotate_pairs(q[:, :, d:], positions, f, magnitude)
        if m.get("kv_from") is None:
            kept[i] = self.latent(i, m, h, positions)
        c, k_rot = kept[i if m.get("kv_from") is None else m["kv_from"]]
        k_plain = (c @ self.t(f"{p}.uk").T).reshape(n, heads, d)
        v = (c @ self.t(f"{p}.uv").T).reshape(n, heads, dv)
        q_all = torch.cat([q[:, :, :d], q_rot], dim=-1)
        k_all = torch.cat([k_plain, k_rot[:, None, :].expand(n, heads, rot)], dim=-1)
        size = m["mask"]["size"] if m.get("mask") else None
        o = softmax_attention(q_all, k_all, v, float(m["scale"]), in_window(n, size), sink=self.t(f"{p}.sink"))
        return o.reshape(n, heads * dv) @ self.t(f"{p}.o").T

    def delta(self, i, m, h, positions):
        p = f"l{i}.mix"
        n = h.shape[0]
        heads, groups, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        q = silu(short_convolution(h @ self.t(f"{p}.q").T, self.t(f"{p}.q.conv"))).reshape(n, groups, d)
        k = silu(short_convolution(h @ self.t(f"{p}.k").T, self.t(f"{p}.k.conv"))).reshape(n, groups, d)
        v = silu(short_convolution(h @ self.t(f"{p}.v").T, self.t(f"{p}.v.conv"))).reshape(n, heads, dv)
        q = q / torch.sqrt((q * q).sum(dim=-1, keepdim=True) + 1e-6) * d ** -0.5
        k = k / torch.sqrt((k * k).sum(dim=-1, keepdim=True) + 1e-6)
        spread = torch.arange(heads) // (heads // groups)
        beta = torch.sigmoid(h @ self.t(f"{p}.b").T)
        decay = torch.exp(-torch.exp(self.t(f"{p}.A_log")) * softplus(h @ self.t(f"{p}.a").T + self.t(f"{p}.dt_bias")))
        o = gated_delta_rule(q[:, spread], k[:, spread], v, beta, decay)
        o = rms(o, self.eps) * self.t(f"{p}.norm") * silu(h @ self.t(f"{p}.g").T).reshape(n, heads, dv)
        return o.reshape(n, heads * dv) @ self.t(f"{p}.o").T

    def mixer(self, i, layer, h, positions, kept):
        if layer["type"] == "attention":
            return self.attention(i, layer["mixer"], h, positions)
        if layer["type"] == "latent_attention":
            return self.latent_attention(i, layer["mixer"], h, positions, kept)
        if layer["type"] == "delta":
            return self.delta(i, layer["mixer"], h, positions)
        raise ValueError(layer["type"])

    def feed_forward(self, i, mlp, h, tokens):
        p = f"l{i}.mlp"
        experts = [(self.t(f"{p}.e{e}.gate"), self.t(f"{p}.e{e}.up"), self.t(f"{p}.e{e}.down"))
                   for e in range(mlp["router"]["experts"])]
        return tabled_experts(h, tokens, self.t(f"{p}.table"), experts)

    # -- the whole model ----------------------------------------------------------------------------
    def forward(self, tokens, layers_out=None):
        """Logits [T, vocab] of a whole sequence; ``layers_out`` (a list) receives the residual stream
        (the sum of the streams) after every layer."""
        tokens = torch.as_tensor(tokens, dtype=torch.int64)
        n = len(tokens)
        positions = torch.arange(n)
        x = self.t("embed")[tokens] * float(self.c["embedding"]["scale"])
        s = self.streams
        X = x[:, None, :].repeat(1, s, 1) if s else None
        kept = {}
        for i, layer in enumerate(self.c["layers"]):
            halves = [(1, lambda h: self.mixer(i, layer, h, positions, kept))]
            if layer.get("mlp") is not None:
                halves.append((2, lambda h: self.feed_forward(i, layer["mlp"], h, tokens)))
            for half, run in halves:
                norm = self.t(f"l{i}.norm{half}")
                if s:
                    hc = f"l{i}.hc{half}"
                    y = run(centred_norm(read_streams(X, self.t(f"{hc}.in")), norm, self.eps))
                    X = write_streams(X, y, self.t(f"{hc}.mix"), self.t(f"{hc}.out"))
                else:
                    x = x + run(centred_norm(x, norm, self.eps))
            if layers_out is not None:
                layers_out.append(X.sum(dim=1) if s else x.clone())
        if s:
            x = X.sum(dim=1)
        return centred_norm(x, self.t("final.norm"), self.eps) @ self.t("head").T

    def generate_greedy(self, prompt, n_new):
        tokens = list(prompt)
        for _ in range(n_new):
            tokens.append(int(torch.argmax(self.forward(tokens)[-1])))
        return tokens[len(prompt):]
