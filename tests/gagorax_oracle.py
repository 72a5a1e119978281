"""Slow, plain Gagorax: one token at a time, float64, one function per
mechanism, written from the design's equations only.

This is the oracle the tests compare the engine against. It shares no code
with arks_amd: every recurrence is a Python loop over tokens, attention keeps
a plain list of keys and values, and nothing is batched, paged or chunked.

Weights are a dict name -> tensor (any float dtype; cast to float64 here);
the config is the parsed config.json dict.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square (eps inside the root)."""
    return x / torch.sqrt((x * x).mean() + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


def rotate_pairs_interleaved(v: torch.Tensor, pos: float, base: float,
                             ndims: int) -> torch.Tensor:
    """Turn pairs (2i, 2i+1), i < ndims/2, of a vector by pos * base^(-2i/ndims).
    Dimensions >= ndims pass through."""
    i = torch.arange(ndims // 2, dtype=F64)
    a = pos * torch.pow(torch.tensor(base, dtype=F64), -2.0 * i / ndims)
    c, s = torch.cos(a), torch.sin(a)
    out = v.clone()
    u, w = v[0:ndims:2], v[1:ndims:2]
    out[0:ndims:2] = u * c - w * s
    out[1:ndims:2] = w * c + u * s
    return out


# ---------------------------------------------------------------- mixers
def attention_token(h, pos, st, W, m, eps):
    """Softmax attention with a value-less sink of score 0, per-head q/k unit
    norm, interleaved rotary on q/k and position-rotated values."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    base, rd = m["rot"]["base"], m["rot"]["dims"]
    q = (W["q"] @ h).view(H, D)
    k = (W["k"] @ h).view(G, D)
    v = (W["v"] @ h).view(G, V)
    keys, vals = [], []
    for g in range(G):
        kk = rms_unit(k[g], eps) * W["k.norm"]
        keys.append(rotate_pairs_interleaved(kk, pos, base, rd))
        vals.append(rotate_pairs_interleaved(v[g], pos, base, V))
    st.setdefault("k", []).append(torch.stack(keys))
    st.setdefault("v", []).append(torch.stack(vals))
    K = torch.stack(st["k"])  # [pos+1, G, D]
    Vv = torch.stack(st["v"])  # [pos+1, G, V]
    out = torch.zeros(H, V, dtype=F64)
    rep = H // G
    for hh in range(H):
        g = hh // rep
        qq = rms_unit(q[hh], eps) * W["q.norm"]
        qq = rotate_pairs_interleaved(qq, pos, base, rd)
        s = (K[:, g] @ qq) * m["scale"]  # every j <= pos
        e = torch.exp(s)
        p = e / (1.0 + e.sum())
        acc = p @ Vv[:, g]
        out[hh] = rotate_pairs_interleaved(acc, -pos, base, V)
    return W["o"] @ out.reshape(-1)


def lightning_token(h, pos, st, W, m, eps):
    """Linear attention with a per-head scalar decay and a d x v state."""
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(W["q"] @ h).view(H, D)
    k = silu(W["k"] @ h).view(H, D)
    v = silu(W["v"] @ h).view(H, V)
    if "S" not in st:
        st["S"] = torch.zeros(H, D, V, dtype=F64)
    o = torch.zeros(H, V, dtype=F64)
    for hh in range(H):
        st["S"][hh] = m["decay"][hh] * st["S"][hh] + torch.outer(k[hh], v[hh])
        o[hh] = st["S"][hh].t() @ q[hh]
    y = rms_unit(o.reshape(-1), eps) * W["norm"]
    y = y * torch.sigmoid(W["g"] @ h)
    return W["o"] @ y


def mamba1_token(h, pos, st, W, m, eps):
    """Selective scan with a short causal convolution in front."""
    inner, N, R, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
    xz = W["in"] @ h
    x, z = xz[:inner], xz[inner:]
    if "conv" not in st:
        st["conv"] = [torch.zeros(inner, dtype=F64) for _ in range(taps - 1)]
        st["S"] = torch.zeros(inner, N, dtype=F64)
    window = st["conv"] + [x]
    xc = W["conv.b"].clone()
    for t in range(taps):
        xc = xc + W["conv"][:, t] * window[t]
    st["conv"] = window[1:]
    xc = silu(xc)
    dbc = W["x"] @ xc
    dt, B, C = dbc[:R], dbc[R:R + N], dbc[R + N:]
    dt = softplus(W["dt"] @ dt + W["dt.b"])
    A = -torch.exp(W["A_log"])
    y = torch.zeros(inner, dtype=F64)
    for c in range(inner):
        st["S"][c] = torch.exp(dt[c] * A[c]) * st["S"][c] + dt[c] * xc[c] * B
        y[c] = (st["S"][c] * C).sum() + W["D"][c] * xc[c]
    y = y * silu(z)
    return W["o"] @ y


MIXERS = {"attention": attention_token, "lightning": lightning_token,
          "mamba1": mamba1_token}


def dense_ff(h, W):
    return W["down"] @ gelu_tanh(W["up"] @ h)


# ---------------------------------------------------------------- model
class Oracle:
    def __init__(self, config: dict, weights: dict):
        self.cfg = config
        self.w = {k: v.to(F64) for k, v in weights.items()}
        self.eps = config["norm"]["eps"]

    def sub(self, prefix: str) -> dict:
        n = len(prefix)
        return {k[n:]: v for k, v in self.w.items() if k.startswith(prefix)}

    def new_state(self) -> dict:
        return {"pos": 0,
                "layers": [{"mix": {}} for _ in self.cfg["layers"]]}

    def token(self, state: dict, tok: int, residuals: list | None = None):
        """Feed one token; returns its logits (float64 [vocab])."""
        w, eps = self.w, self.eps
        pos = state["pos"]
        x = w["embed"][tok].clone()
        for i, layer in enumerate(self.cfg["layers"]):
            st = state["layers"][i]
            p = f"l{i}."
            # token shift on the mixer's input only
            prev = st.get("prev", torch.zeros_like(x))
            st["prev"] = x.clone()
            hs = x + (prev - x) * w[p + "shift"]
            y = MIXERS[layer["type"]](hs, pos, st["mix"], self.sub(p + "mix."),
                                      layer["mixer"], eps)
            y = y * torch.sigmoid(w[p + "rg1"] @ x + w[p + "rg1.b"])
            x = x + rms_unit(y, eps) * w[p + "norm1"]
            if layer.get("mlp") is not None:
                assert layer["mlp"]["kind"] == "dense"
                y = dense_ff(x, self.sub(p + "mlp."))
                y = y * torch.sigmoid(w[p + "rg2"] @ x + w[p + "rg2.b"])
                x = x + rms_unit(y, eps) * w[p + "norm2"]
            if residuals is not None:
                residuals.append(x.clone())
        state["pos"] = pos + 1
        xf = rms_unit(x, eps) * w["final.norm"]
        return (w["head"] @ xf) * self.cfg["logit_scale"]

    def run(self, tokens: list[int]) -> torch.Tensor:
        st = self.new_state()
        return torch.stack([self.token(st, t) for t in tokens])


def random_weights(config: dict, seed: int = 0, dtype=torch.bfloat16) -> dict:
    """Random tensors of the design's names and shapes for a config."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = config["width"], config["vocab"]

    def rn(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    out = {"embed": rn(V, Wd), "head": rn(V, Wd, std=Wd ** -0.5),
           "final.norm": 1.0 + rn(Wd, std=0.1)}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = 1.0 + rn(Wd, std=0.1)
        out[p + "shift"] = torch.rand(Wd, generator=g).to(dtype)
        out[p + "rg1"] = rn(Wd, Wd, std=Wd ** -0.5)
        out[p + "rg1.b"] = rn(Wd, std=0.5)
        t = layer["type"]
        if t == "attention":
            H, G, D, Vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out[p + "mix.q"] = rn(H * D, Wd, std=Wd ** -0.5)
            out[p + "mix.k"] = rn(G * D, Wd, std=Wd ** -0.5)
            out[p + "mix.v"] = rn(G * Vd, Wd, std=Wd ** -0.5)
            out[p + "mix.q.norm"] = 1.0 + rn(D, std=0.2)
            out[p + "mix.k.norm"] = 1.0 + rn(D, std=0.2)
            out[p + "mix.o"] = rn(Wd, H * Vd, std=(H * Vd) ** -0.5)
        elif t == "lightning":
            H, D, Vd = m["heads"], m["dim"], m["vdim"]
            out[p + "mix.q"] = rn(H * D, Wd, std=Wd ** -0.5)
            out[p + "mix.k"] = rn(H * D, Wd, std=Wd ** -0.5)
            out[p + "mix.v"] = rn(H * Vd, Wd, std=Wd ** -0.5)
            out[p + "mix.g"] = rn(H * Vd, Wd, std=Wd ** -0.5)
            out[p + "mix.norm"] = 1.0 + rn(H * Vd, std=0.1)
            out[p + "mix.o"] = rn(Wd, H * Vd, std=(H * Vd) ** -0.5)
        elif t == "mamba1":
            inner, N, R, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
            out[p + "mix.in"] = rn(2 * inner, Wd, std=Wd ** -0.5)
            out[p + "mix.conv"] = rn(inner, taps, std=taps ** -0.5)
            out[p + "mix.conv.b"] = rn(inner, std=0.1)
            out[p + "mix.x"] = rn(R + 2 * N, inner, std=inner ** -0.5)
            out[p + "mix.dt"] = rn(inner, R, std=R ** -0.5)
            out[p + "mix.dt.b"] = rn(inner, std=0.5) - 2.0
            out[p + "mix.A_log"] = torch.log(
                1.0 + 3.0 * torch.rand(inner, N, generator=g)).to(dtype)
            out[p + "mix.D"] = rn(inner, std=0.5)
            out[p + "mix.o"] = rn(Wd, inner, std=inner ** -0.5)
        else:
            raise ValueError(t)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out[p + "norm2"] = 1.0 + rn(Wd, std=0.1)
            out[p + "mlp.up"] = rn(ff, Wd, std=Wd ** -0.5)
            out[p + "mlp.down"] = rn(Wd, ff, std=ff ** -0.5)
            out[p + "rg2"] = rn(Wd, Wd, std=Wd ** -0.5)
            out[p + "rg2.b"] = rn(Wd, std=0.5)
    return out
