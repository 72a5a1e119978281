"""A slow float64 model of the Fusolix design, one function per mechanism,
written from the design's equations and sharing nothing with arks_amd.

A model is (cfg, weights): cfg the dict of config.json, weights a dict of
float64 tensors by checkpoint name. forward() runs one whole sequence and
returns the logits of every position (and the summed streams after every
layer); there is no cache: every position looks back over the full prefix,
the recurrences start from zero at position 0.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def short_conv_residual(h, w):
    """h [n, C], w [C, taps]: h_t + sum_j w[:, j] h_(t - taps + 1 + j)."""
    n, _ = h.shape
    taps = w.shape[1]
    out = h.clone()
    for t in range(n):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


def streams_read(xs, w_in):
    """xs [s, n, C] -> [n, C]."""
    return torch.einsum("s,snc->nc", w_in, xs)


def streams_write(xs, y, w_mix, w_out):
    """new[t] = sum_s mix[s, t] old[s] + out[t] y."""
    return torch.einsum("st,snc->tnc", w_mix, xs) + w_out[:, None, None] * y[None]


def window_pool_attention(q, k, v, scale, window, pool):
    """q [n, H, D], k [n, G, D], v [n, G, V]. Row i sees the keys j with
    0 <= i - j < window, and the mean key / mean value of every block of
    `pool` consecutive positions whose last position is <= i - window."""
    n, H, D = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(n, H, v.shape[2], dtype=F64)
    for i in range(n):
        lo = max(0, i - window + 1)
        nblk = max(0, (i - window + 1) // pool) if i - window + 1 >= 0 else 0
        keys = [k[b * pool:(b + 1) * pool].mean(0) for b in range(nblk)]
        vals = [v[b * pool:(b + 1) * pool].mean(0) for b in range(nblk)]
        keys += [k[j] for j in range(lo, i + 1)]
        vals += [v[j] for j in range(lo, i + 1)]
        K = torch.stack(keys)  # [m, G, D]
        Vv = torch.stack(vals)
        for h in range(H):
            g = h // rep
            s = (K[:, g] @ q[i, h]) * scale
            p = torch.softmax(s, 0)
            out[i, h] = p @ Vv[:, g]
    return out


def rotate_half_split(x, pos, base, dims):
    """x [n, H, D]: the first `dims` dims of every head turn, dim i paired
    with dim i + dims/2, by the angle pos * base^(-2i/dims)."""
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    f = torch.tensor(float(base), dtype=F64) ** (-2.0 * i / dims)
    a = pos.to(F64)[:, None, None] * f[None, None, :]
    c, s = torch.cos(a), torch.sin(a)
    u, w = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * c - w * s
    out[..., half:dims] = w * c + u * s
    return out


def retention(q, k, v, decay):
    """q, k [n, H, D], v [n, H, V]: S <- decay_h S + k v^T, o = S^T q."""
    n, H, D = q.shape
    V = v.shape[2]
    S = torch.zeros(H, D, V, dtype=F64)
    lam = torch.tensor([float(d) for d in decay], dtype=F64)[:, None, None]
    out = torch.zeros(n, H, V, dtype=F64)
    for t in range(n):
        S = lam * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def unit_rms(x, eps):
    return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps)


def parallel_mixer(h, m, w, pre, eps):
    """h [n, C]; m the mixer's config; w the weights; pre the name prefix."""
    n = h.shape[0]
    L, R = m["left"], m["right"]
    lp, rp = pre + "left.", pre + "right."
    q = (h @ w[lp + "q"].T + w[lp + "q.b"]).view(n, L["heads"], L["dim"])
    k = (h @ w[lp + "k"].T + w[lp + "k.b"]).view(n, L["kv_heads"], L["dim"])
    v = (h @ w[lp + "v"].T + w[lp + "v.b"]).view(n, L["kv_heads"], L["vdim"])
    a = window_pool_attention(q, k, v, L["scale"], L["mask"]["size"],
                              L["mask"]["pool"])
    left = a.reshape(n, -1) @ w[lp + "o"].T + w[lp + "o.b"]

    pos = torch.arange(n)
    q = (h @ w[rp + "q"].T).view(n, R["heads"], R["dim"])
    k = (h @ w[rp + "k"].T).view(n, R["heads"], R["dim"])
    v = (h @ w[rp + "v"].T).view(n, R["heads"], R["vdim"])
    q = rotate_half_split(q, pos, R["rot"]["base"], R["rot"]["dims"])
    k = rotate_half_split(k, pos, R["rot"]["base"], R["rot"]["dims"])
    k = k * R["dim"] ** -0.5
    o = unit_rms(retention(q, k, v, R["decay"]), eps).reshape(n, -1)
    gate = h @ w[rp + "g"].T
    right = (o * gate * torch.sigmoid(gate)) @ w[rp + "o"].T
    return m["left_scale"] * left + m["right_scale"] * right


def clamped_glu(h, mlp, w, pre):
    lim = mlp["limit"]
    g = torch.clamp(h @ w[pre + "gate"].T, max=lim)
    u = torch.clamp(h @ w[pre + "up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def route(z, top, groups, keep):
    """z [E] router logits -> (expert ids, weights)."""
    s = torch.softmax(z, 0)
    E = s.shape[0]
    per = E // groups
    gscore = s.view(groups, per).max(1).values
    kept = torch.topk(gscore, keep).indices.tolist()
    allowed = torch.full((E,), -1.0, dtype=F64)
    for g in kept:
        allowed[g * per:(g + 1) * per] = s[g * per:(g + 1) * per]
    ids = torch.topk(allowed, top).indices
    wts = s[ids]
    return ids.tolist(), (wts / (wts.sum() + 1e-20)).tolist()


def grouped_moe(h, mlp, w, pre):
    r = mlp["router"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        z = w[pre + "router"] @ h[t]
        ids, wts = route(z, r["top"], r["groups"]["count"], r["groups"]["keep"])
        for e, c in zip(ids, wts):
            p = f"{pre}e{e}."
            a = w[p + "gate"] @ h[t]
            y = (a * torch.sigmoid(a)) * (w[p + "up"] @ h[t])
            out[t] += c * (w[p + "down"] @ y)
    return out


def forward(cfg, w, tokens):
    """-> (logits [n, vocab], [layer sums [n, C]])."""
    eps = cfg["norm"]["eps"]
    s = cfg["streams"]
    x0 = w["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    xs = torch.stack([x0] * s)
    sums = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        assert layer["type"] == "parallel"
        u = streams_read(xs, w[p + "hc1.in"])
        h = layer_norm(u, w[p + "norm1"], w[p + "norm1.b"], eps)
        h = short_conv_residual(h, w[p + "canon1"])
        y = parallel_mixer(h, layer["mixer"], w, p + "mix.", eps)
        xs = streams_write(xs, y, w[p + "hc1.mix"], w[p + "hc1.out"])
        mlp = layer.get("mlp")
        if mlp is not None:
            u = streams_read(xs, w[p + "hc2.in"])
            h = layer_norm(u, w[p + "norm2"], w[p + "norm2.b"], eps)
            h = short_conv_residual(h, w[p + "canon2"])
            if mlp["kind"] == "dense":
                y = clamped_glu(h, mlp, w, p + "mlp.")
            else:
                y = grouped_moe(h, mlp, w, p + "mlp.")
            xs = streams_write(xs, y, w[p + "hc2.mix"], w[p + "hc2.out"])
        sums.append(xs.sum(0))
    x = layer_norm(xs.sum(0), w["final.norm"], w["final.norm.b"], eps)
    return x @ w["head"].T, sums


# ---------------------------------------------------------------- test models
def tensor_shapes(cfg) -> dict:
    C, s, taps = cfg["width"], cfg["streams"], cfg["canon"]["taps"]
    sh = {"embed": (cfg["vocab"], C), "head": (cfg["vocab"], C),
          "final.norm": (C,), "final.norm.b": (C,)}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        L, R = layer["mixer"]["left"], layer["mixer"]["right"]
        sh.update({
            p + "norm1": (C,), p + "norm1.b": (C,), p + "canon1": (C, taps),
            p + "hc1.in": (s,), p + "hc1.out": (s,), p + "hc1.mix": (s, s),
            p + "mix.left.q": (L["heads"] * L["dim"], C),
            p + "mix.left.q.b": (L["heads"] * L["dim"],),
            p + "mix.left.k": (L["kv_heads"] * L["dim"], C),
            p + "mix.left.k.b": (L["kv_heads"] * L["dim"],),
            p + "mix.left.v": (L["kv_heads"] * L["vdim"], C),
            p + "mix.left.v.b": (L["kv_heads"] * L["vdim"],),
            p + "mix.left.o": (C, L["heads"] * L["vdim"]),
            p + "mix.left.o.b": (C,),
            p + "mix.right.q": (R["heads"] * R["dim"], C),
            p + "mix.right.k": (R["heads"] * R["dim"], C),
            p + "mix.right.v": (R["heads"] * R["vdim"], C),
            p + "mix.right.g": (R["heads"] * R["vdim"], C),
            p + "mix.right.o": (C, R["heads"] * R["vdim"]),
        })
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        sh.update({p + "norm2": (C,), p + "norm2.b": (C,),
                   p + "canon2": (C, taps), p + "hc2.in": (s,),
                   p + "hc2.out": (s,), p + "hc2.mix": (s, s)})
        if mlp["kind"] == "dense":
            sh.update({p + "mlp.gate": (mlp["ff"], C), p + "mlp.up": (mlp["ff"], C),
                       p + "mlp.down": (C, mlp["ff"])})
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            sh[p + "mlp.router"] = (E, C)
            for e in range(E):
                sh.update({f"{p}mlp.e{e}.gate": (ff, C), f"{p}mlp.e{e}.up": (ff, C),
                           f"{p}mlp.e{e}.down": (C, ff)})
    return sh


def random_weights(cfg, seed: int, dtype=torch.bfloat16) -> dict:
    """Random weights with activations of order one; values are rounded to
    `dtype` (what a checkpoint would hold) and returned in float64."""
    g = torch.Generator().manual_seed(seed)
    s = cfg["streams"]
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name[0] == "l" and name[1].isdigit() else name
        rn = lambda std: torch.randn(shape, generator=g, dtype=F64) * std
        if leaf in ("norm1", "norm2", "final.norm"):
            t = 1.0 + rn(0.1)
        elif leaf.endswith(".b"):
            t = rn(0.2)
        elif leaf.startswith("canon"):
            t = rn(0.3)
        elif leaf.endswith(".in"):
            t = 1.0 / s + rn(0.2)
        elif leaf.endswith(".out"):
            t = 1.0 + rn(0.3)
        elif leaf.endswith(".mix"):
            t = torch.eye(s, dtype=F64) + rn(0.15)
        elif leaf == "embed":
            t = rn(1.0 / cfg["embedding"]["scale"])
        elif leaf.endswith("router"):
            t = rn(2.0 * shape[-1] ** -0.5)
        else:
            t = rn(shape[-1] ** -0.5)
        out[name] = t.to(dtype).to(F64)
    return out


def make_config(*, vocab=96, width=48, streams=2, taps=3, eps=1e-5,
                embed_scale=3.0, layers=("dense", "moe"), heads=4, kv_heads=2,
                dim=16, vdim=16, scale=0.3, window=8, pool=4, r_heads=2,
                r_dim=16, r_vdim=8, decay=(0.9, 0.97), rot_dims=8,
                rot_base=100.0, left_scale=0.8, right_scale=1.1, ff=64,
                limit=2.0, experts=6, top=2, groups=3, keep=2, expert_ff=24):
    """A small config of the design; `layers` names each layer's
    feed-forward: "dense", "moe" or None."""
    out = []
    for kind in layers:
        mixer = {
            "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                     "vdim": vdim, "scale": scale,
                     "mask": {"size": window, "pool": pool}},
            "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim,
                      "decay": list(decay)[:r_heads],
                      "rot": {"base": rot_base, "dims": rot_dims}},
            "left_scale": left_scale, "right_scale": right_scale}
        if kind == "dense":
            mlp = {"kind": "dense", "ff": ff, "limit": limit}
        elif kind == "moe":
            mlp = {"kind": "moe", "expert": {"ff": expert_ff},
                   "router": {"experts": experts, "top": top,
                              "groups": {"count": groups, "keep": keep}}}
        else:
            mlp = None
        out.append({"type": "parallel", "mixer": mixer, "mlp": mlp})
    return {"architecture": "Fusolix", "vocab": vocab, "width": width,
            "streams": streams, "canon": {"taps": taps},
            "embedding": {"scale": embed_scale}, "norm": {"eps": eps},
            "layers": out}
