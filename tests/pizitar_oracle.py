"""Plain, slow restatement of the Pizitar decoder (CPU, float64 by default), one function per mechanism.

Shares no code with ming_univision_amd: it reads a configuration dict (the keys of the model's config.json) and a
{tensor name: torch tensor} dict, and evaluates whole sequences at once.  Tests compare the HIP path against it.

Notation: x [T, W] is the residual stream of ONE sequence, t the position (from 0), W the width.
"""
import math

import torch

DT = torch.float64


def affine_layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(var + eps) * w + b with the biased variance of every row."""
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) per row."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * w


def causal_tap_filter(h, w):
    """h [T, W], w [W, taps]: y_t = sum_j w[:, j] * h_(t - taps + 1 + j), rows before the start are zero."""
    T, taps = h.shape[0], w.shape[1]
    y = torch.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * h[s]
    return y


def sigmoid_gate(h, w, b):
    return torch.sigmoid(h @ w.T + b)


def poly_norm(z, coef, eps):
    """coef = (a, b, c, e): a U(z) + b U(z^2) + c U(z^3) + e, U = rms_unit over the row."""
    a, b, c, e = [coef[i] for i in range(4)]
    return a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e


def dense_ff(h, up, down, coef, eps):
    return poly_norm(h @ up.T, coef, eps) @ down.T


def latent_of(h, w_dkv, w_norm, eps):
    """The cached quantity of a latent-attention layer: rms_norm(W_dkv h)."""
    return rms_norm(h @ w_dkv.T, w_norm, eps)


def latent_attention_core(q, c, w_uk, w_uv, heads, dim, vdim, scale):
    """q [T, heads*dim], c [T, r] latents of the SAME positions; keys / values of head n are rows n*dim.. of W_uk c and
    n*vdim.. of W_uv c; causal softmax.  Returns [T, heads*vdim].  Written key by key, no matrix tricks."""
    T = q.shape[0]
    k = c @ w_uk.T
    v = c @ w_uv.T
    out = torch.zeros(T, heads * vdim, dtype=q.dtype)
    for n in range(heads):
        qn, kn, vn = q[:, n * dim:(n + 1) * dim], k[:, n * dim:(n + 1) * dim], v[:, n * vdim:(n + 1) * vdim]
        for t in range(T):
            s = (kn[:t + 1] @ qn[t]) * scale
            p = torch.softmax(s, 0)
            out[t, n * vdim:(n + 1) * vdim] = p @ vn[:t + 1]
    return out


def mixer_latent_attention(h, P, m, eps, shared_latent=None):
    """Queries through a normed low-rank latent; returns (output [T, W], latent c [T, r])."""
    cq = rms_norm(h @ P["dq"].T, P["dq.norm"], eps)
    q = cq @ P["uq"].T
    c = shared_latent if shared_latent is not None else latent_of(h, P["dkv"], P["dkv.norm"], eps)
    o = latent_attention_core(q, c, P["uk"], P["uv"], m["heads"], m["dim"], m["vdim"], m["scale"])
    return o @ P["o"].T, c


def mixer_latent_attention_2(h, P, m, eps):
    """Direct queries and a sigmoid gate on the concatenated heads."""
    q = h @ P["q"].T
    c = latent_of(h, P["dkv"], P["dkv.norm"], eps)
    o = latent_attention_core(q, c, P["uk"], P["uv"], m["heads"], m["dim"], m["vdim"], m["scale"])
    o = o * torch.sigmoid(h @ P["g"].T)
    return o @ P["o"].T, c


def layer_params(sd, i, kind):
    pre = f"l{i}.{kind}."
    return {k[len(pre):]: v for k, v in sd.items() if k.startswith(pre)}


def run_layers(cfg, sd, tokens, dtype=DT, trace=None):
    """Whole sequence through every layer -> residual stream [T, W]; trace (a list) receives the stream after every layer."""
    sd = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x = sd["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    latents = {}
    for i, ly in enumerate(cfg["layers"]):
        p = f"l{i}."
        n1 = affine_layer_norm(x, sd[p + "norm1"], sd[p + "norm1.b"], eps)
        g1 = sigmoid_gate(n1, sd[p + "rg1"], sd[p + "rg1.b"])
        h = n1 + causal_tap_filter(n1, sd[p + "canon1"])
        P, m = layer_params(sd, i, "mix"), ly["mixer"]
        if ly["type"] == "latent_attention":
            src = m.get("kv_from")
            y, c = mixer_latent_attention(h, P, m, eps, None if src is None else latents[src])
        elif ly["type"] == "latent_attention_2":
            y, c = mixer_latent_attention_2(h, P, m, eps)
        else:
            raise ValueError(ly["type"])
        latents[i] = c
        x = x + affine_layer_norm(g1 * y, sd[p + "norm1b"], sd[p + "norm1b.b"], eps)
        if ly.get("mlp") is not None:
            assert ly["mlp"]["kind"] == "dense"
            n2 = affine_layer_norm(x, sd[p + "norm2"], sd[p + "norm2.b"], eps)
            g2 = sigmoid_gate(n2, sd[p + "rg2"], sd[p + "rg2.b"])
            F = layer_params(sd, i, "mlp")
            y = dense_ff(n2, F["up"], F["down"], F["act"], eps)
            x = x + affine_layer_norm(g2 * y, sd[p + "norm2b"], sd[p + "norm2b.b"], eps)
        if trace is not None:
            trace.append(x.clone())
    return x, sd


def logits_of(cfg, sd, tokens, dtype=DT, trace=None):
    """[T, vocab] logits of one sequence, soft-capped."""
    x, sd = run_layers(cfg, sd, tokens, dtype, trace)
    y = affine_layer_norm(x, sd["final.norm"], sd["final.norm.b"], cfg["norm"]["eps"])
    z = y @ sd["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


# ---- random models for tests ----------------------------------------------------------------------------------------------
def random_config(layers, width=48, vocab=67, taps=3, eps=1e-5, softcap=20.0):
    """layers: list of dicts(type=..., heads, dim, vdim, kv_rank, [q_rank], [kv_from], ff (None = no feed-forward))."""
    out = []
    for ly in layers:
        m = {k: ly[k] for k in ("heads", "dim", "vdim", "kv_rank") }
        m["scale"] = ly.get("scale", 1.0 / math.sqrt(ly["dim"]))
        if ly["type"] == "latent_attention":
            m["q_rank"] = ly["q_rank"]
            if ly.get("kv_from") is not None:
                m["kv_from"] = ly["kv_from"]
        out.append({"type": ly["type"], "mixer": m, "mlp": None if ly.get("ff") is None else {"kind": "dense", "ff": ly["ff"]}})
    return {"architecture": "Pizitar", "canon": {"taps": taps}, "layers": out, "logit_softcap": softcap, "norm": {"eps": eps},
            "vocab": vocab, "width": width}


def tensor_shapes(cfg):
    W, V, taps = cfg["width"], cfg["vocab"], cfg["canon"]["taps"]
    sh = {"embed": (V, W), "final.norm": (W,), "final.norm.b": (W,), "head": (V, W)}
    for i, ly in enumerate(cfg["layers"]):
        p, m = f"l{i}.", ly["mixer"]
        has_ff = ly.get("mlp") is not None
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if has_ff else ()):
            sh[p + n] = (W,)
            sh[p + n + ".b"] = (W,)
        H, d, v, r = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
        if ly["type"] == "latent_attention":
            sh[p + "mix.dq"], sh[p + "mix.dq.norm"], sh[p + "mix.uq"] = (m["q_rank"], W), (m["q_rank"],), (H * d, m["q_rank"])
        else:
            sh[p + "mix.q"], sh[p + "mix.g"] = (H * d, W), (H * v, W)
        if m.get("kv_from") is None:
            sh[p + "mix.dkv"], sh[p + "mix.dkv.norm"] = (r, W), (r,)
        sh[p + "mix.uk"], sh[p + "mix.uv"], sh[p + "mix.o"] = (H * d, r), (H * v, r), (W, H * v)
        if ly.get("mlp") is not None:
            ff = ly["mlp"]["ff"]
            sh[p + "mlp.up"], sh[p + "mlp.down"], sh[p + "mlp.act"] = (ff, W), (W, ff), (4,)
        sh[p + "canon1"] = (W, taps)
        for n in ("rg1",) + (("rg2",) if has_ff else ()):
            sh[p + n], sh[p + n + ".b"] = (W, W), (W,)
    return sh


def random_weights(cfg, seed=0, gain=1.0):
    """bf16-valued random tensors (what a checkpoint holds), norm weights near 1."""
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for k, s in tensor_shapes(cfg).items():
        last = k.split(".")[-1]
        if k.endswith("mlp.act"):
            t = torch.tensor([0.6, 0.3, 0.2, 0.05]) + 0.1 * torch.randn(4, generator=g)
        elif last == "b":
            t = 0.1 * torch.randn(s, generator=g)
        elif len(s) == 1:
            t = 1.0 + 0.2 * torch.randn(s, generator=g)
        elif last == "canon1":
            t = 0.4 * torch.randn(s, generator=g)
        elif k == "embed":
            t = torch.randn(s, generator=g)
        else:
            t = gain * torch.randn(s, generator=g) * s[-1] ** -0.5
        sd[k] = t.to(torch.bfloat16)
    return sd
