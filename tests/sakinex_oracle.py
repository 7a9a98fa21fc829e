"""Plain, slow restatement of the Sakinex decoder (CPU, float64 by default), one function per mechanism.

Shares no code with ming_univision_amd: it reads a configuration dict (the keys of the model's config.json) and a
{tensor name: torch tensor} dict, and evaluates whole sequences at once, position by position where that is the clearest form.
Tests compare the HIP path against it.

Notation: x [T, W] is the residual stream of ONE sequence, t the position (from 0), W the width.
"""
import math

import torch

DT = torch.float64


# ---- norms, filters ---------------------------------------------------------------------------------------------------------------
def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * w


def causal_taps(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] * u_(t - taps + 1 + j); inputs before the sequence's start are zero."""
    T, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] = y[t] + w[:, j] * u[s]
    return y


def sublayer_input(n, w):
    """What a sublayer reads: its normed input plus the causal per-channel filter of it (w None: no filter)."""
    return n if w is None else n + causal_taps(n, w)


# ---- rotary positions -------------------------------------------------------------------------------------------------------------
def rotary_frequencies(rot):
    """-> (frequency of every rotated pair [dims / 2], magnitude factor of cos and sin)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=DT), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=DT), 0.1 * math.log(factor) + 1.0


def rotate(u, pos, rot):
    """u [T, heads, dim]; the first rot.dims values of every head are rotated in pairs (i, i + dims / 2), the rest pass."""
    if not rot:
        return u
    dims = int(rot["dims"])
    half = dims // 2
    freq, mag = rotary_frequencies(rot)
    ang = pos.to(DT)[:, None] * freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = u[..., :half], u[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, u[..., dims:]], -1)


# ---- left mixer: windowed attention with pooled blocks ---------------------------------------------------------------------------
def visible(i, mask):
    """-> (token positions, pooled blocks) that position i sees.  mask None: every earlier token and itself."""
    if not mask:
        return list(range(i + 1)), []
    size = int(mask["size"])
    toks = [j for j in range(i + 1) if i - j < size]
    pool = mask.get("pool")
    blocks = []
    if pool:
        P = int(pool)
        b = 0
        while b * P + P - 1 <= i - size:
            blocks.append(b)
            b += 1
    return toks, blocks


def windowed_attention(q, k, v, scale, mask, rows=None):
    """q [T, H, d], k [T, G, d], v [T, G, e] as the cache holds them -> [T, H, e].  Tokens in the window and the means of the
    whole blocks before it share one softmax.  rows: the positions to evaluate (default all; the others stay zero)."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    P = int(mask["pool"]) if mask and mask.get("pool") else 0
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for i in (range(T) if rows is None else rows):
        toks, blocks = visible(i, mask)
        for h in range(H):
            g = h // rep
            ks = [k[b * P:(b + 1) * P, g].mean(0) for b in blocks] + [k[j, g] for j in toks]
            vs = [v[b * P:(b + 1) * P, g].mean(0) for b in blocks] + [v[j, g] for j in toks]
            ks, vs = torch.stack(ks), torch.stack(vs)
            p = torch.softmax((ks @ q[i, h]) * scale, 0)
            out[i, h] = p @ vs
    return out


def left_mixer(h, sd, p, m, eps):
    """Projections, short filter, rotation, unit norm per head, attention, output projection."""
    H, G, d, e = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q, k, v = h @ sd[p + "q"].T, h @ sd[p + "k"].T, h @ sd[p + "v"].T
    if m.get("conv"):
        q, k, v = causal_taps(q, sd[p + "q.conv"]), causal_taps(k, sd[p + "k.conv"]), causal_taps(v, sd[p + "v.conv"])
    pos = torch.arange(T)
    q = rms_unit(rotate(q.reshape(T, H, d), pos, m.get("rot")), eps)
    k = rms_unit(rotate(k.reshape(T, G, d), pos, m.get("rot")), eps)
    a = windowed_attention(q, k, v.reshape(T, G, e), float(m["scale"]), m.get("mask"))
    return a.reshape(T, H * e) @ sd[p + "o"].T


# ---- right mixer: minGRU ---------------------------------------------------------------------------------------------------------
def gru_candidate(u):
    return torch.where(u >= 0, u + 0.5, torch.sigmoid(u))


def min_gru(h, sd, p):
    z = torch.sigmoid(h @ sd[p + "z"].T + sd[p + "z.b"])
    c = gru_candidate(h @ sd[p + "x"].T + sd[p + "x.b"])
    g = h @ sd[p + "g"].T
    S = torch.zeros(z.shape[1], dtype=h.dtype)
    out = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * c[t]
        out.append(S * (g[t] * torch.sigmoid(g[t])))
    return torch.stack(out) @ sd[p + "o"].T


def parallel_mixer(h, sd, p, m, eps):
    return float(m["left_scale"]) * left_mixer(h, sd, p + "left.", m["left"], eps) + float(m["right_scale"]) * min_gru(h, sd, p + "right.")


# ---- feed-forward: mixture of experts ---------------------------------------------------------------------------------------------
def gated_expert(h, sd, p):
    g = h @ sd[p + "gate"].T
    return ((g * torch.sigmoid(g)) * (h @ sd[p + "up"].T)) @ sd[p + "down"].T


def route(h, sd, p, top):
    """-> (chosen experts [T, top], their weights [T, top]): largest logits, softmax over the chosen logits only."""
    z = h @ sd[p + "router"].T + sd[p + "router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, -1)


def moe(h, sd, p, mlp):
    idx, w = route(h, sd, p, int(mlp["router"]["top"]))
    out = torch.zeros(h.shape[0], sd[p + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            out[t] = out[t] + w[t, j] * gated_expert(h[t:t + 1], sd, f"{p}e{int(idx[t, j])}.")[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ sd[p + "shared.sg"].T) * gated_expert(h, sd, p + "shared.")
    return out


# ---- the stack ------------------------------------------------------------------------------------------------------------------
def layer_runs(cfg):
    """-> [(layer index, first of a repeated pass)]: layers start .. stop - 1 run `times` times in a row, the rest once."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for r in range(times):
        runs += [(i, r > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def layer(x, sd, cfg, i):
    ly, eps, mult = cfg["layers"][i], float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    p = f"l{i}."
    canon = bool(cfg.get("canon"))
    h = sublayer_input(rms_norm(x, sd[p + "norm1"], eps), sd[p + "canon1"] if canon else None)
    x = x + mult * parallel_mixer(h, sd, p + "mix.", ly["mixer"], eps)
    if ly.get("mlp") is not None:
        h = sublayer_input(rms_norm(x, sd[p + "norm2"], eps), sd[p + "canon2"] if canon else None)
        x = x + mult * moe(h, sd, p + "mlp.", ly["mlp"])
    return x


def forward(cfg, sd, ids, trace=False):
    """ids: token list of one sequence -> logits [T, vocab] (and the residual stream after every layer run when trace)."""
    sd = {k: v.to(DT) for k, v in sd.items()}
    e = sd["embed"][torch.as_tensor(ids, dtype=torch.long)]
    x, streams = e, []
    for i, again in layer_runs(cfg):
        if again:
            x = x + e
        x = layer(x, sd, cfg, i)
        streams.append(x)
    logits = rms_norm(x, sd["final.norm"], float(cfg["norm"]["eps"])) @ sd["head"].T
    return (logits, torch.stack(streams)) if trace else logits


# ---- small random models -----------------------------------------------------------------------------------------------------------
def tensor_shapes(cfg):
    W, V = int(cfg["width"]), int(cfg["vocab"])
    taps = int(cfg["canon"]["taps"]) if cfg.get("canon") else 0
    s = {"embed": (V, W)}
    for i, ly in enumerate(cfg["layers"]):
        p, m, mlp = f"l{i}.", ly["mixer"], ly.get("mlp")
        L, R = m["left"], m["right"]
        H, G, d, e = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
        s[p + "norm1"] = (W,)
        for n, rows in (("q", H * d), ("k", G * d), ("v", G * e)):
            s[p + "mix.left." + n] = (rows, W)
            if L.get("conv"):
                s[p + "mix.left." + n + ".conv"] = (rows, L["conv"])
        s[p + "mix.left.o"] = (W, H * e)
        for n in ("z", "x"):
            s[p + "mix.right." + n], s[p + "mix.right." + n + ".b"] = (R["width"], W), (R["width"],)
        s[p + "mix.right.g"], s[p + "mix.right.o"] = (R["width"], W), (W, R["width"])
        if mlp is not None:
            s[p + "norm2"] = (W,)
            ff = mlp["expert"]["ff"]
            for j in range(mlp["router"]["experts"]):
                s[f"{p}mlp.e{j}.gate"], s[f"{p}mlp.e{j}.up"], s[f"{p}mlp.e{j}.down"] = (ff, W), (ff, W), (W, ff)
            s[p + "mlp.router"], s[p + "mlp.router.b"] = (mlp["router"]["experts"], W), (mlp["router"]["experts"],)
            if mlp.get("shared"):
                fs = mlp["shared"]["ff"]
                s[p + "mlp.shared.gate"], s[p + "mlp.shared.up"], s[p + "mlp.shared.down"] = (fs, W), (fs, W), (W, fs)
                s[p + "mlp.shared.sg"] = (1, W)
            if taps:
                s[p + "canon2"] = (W, taps)
        if taps:
            s[p + "canon1"] = (W, taps)
    s["final.norm"], s["head"] = (W,), (V, W)
    return s


def random_weights(cfg, seed=0):
    """bf16 tensors of a size that keeps every activation of order one."""
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for k, shp in tensor_shapes(cfg).items():
        if k.endswith("norm1") or k.endswith("norm2") or k == "final.norm":
            t = 1.0 + 0.1 * torch.randn(shp, generator=g)
        elif k.endswith(".b"):
            t = 0.5 * torch.randn(shp, generator=g)
        elif k.endswith(".conv") or "canon" in k:
            t = 0.4 * torch.randn(shp, generator=g)
        elif k == "embed":
            t = torch.randn(shp, generator=g)
        elif k.endswith("router"):
            t = 2.0 * torch.randn(shp, generator=g) / math.sqrt(shp[-1])
        else:
            t = torch.randn(shp, generator=g) / math.sqrt(shp[-1])
        sd[k] = t.to(torch.bfloat16)
    return sd


def small_config(width=64, vocab=96, n_layers=3, heads=4, kv_heads=2, dim=16, vdim=24, rot_dims=8, conv=3, window=9, pool=4, gru=40,
                 experts=5, top=2, ff=24, shared_ff=16, taps=3, loop=(1, 2, 2), no_mlp=(), scaling=True, eps=1e-5, mult=0.7):
    rot = {"base": 100.0, "dims": rot_dims}
    if scaling:
        rot["scaling"] = {"factor": 4.0, "fast": 8.0, "original": 16, "slow": 1.0}
    layers = []
    for i in range(n_layers):
        left = {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"pool": pool, "size": window}, "rot": rot,
                "scale": 1.3 / math.sqrt(dim), "vdim": vdim}
        mlp = None if i in no_mlp else {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "top": top},
                                        "shared": {"ff": shared_ff}}
        layers.append({"type": "parallel", "mixer": {"left": left, "left_scale": 0.8, "right": {"width": gru}, "right_scale": 0.6}, "mlp": mlp})
    cfg = {"architecture": "Sakinex", "canon": {"taps": taps}, "layers": layers, "norm": {"eps": eps}, "residual_mult": mult,
           "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg
