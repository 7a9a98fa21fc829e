"""Pizitar on the HIP path against tests/pizitar_oracle.py (plain float64 restatement, one function per mechanism).

Small random models of several shapes (never equal head / latent / value sizes unless a test says so), fp32 arithmetic held to 1e-4
of the logits' scale, the bf16-MFMA arithmetic to 3e-2.  Covers: every operator alone; whole prompts; token-by-token decoding;
portions down to two tokens; several unequal requests in one pass against each alone; cache sequences that are released and
reused; keys at and around the edges of the attention kernel's key tiles and key splits, inside and just outside a row's length;
the first positions of a sequence (the causal filter's zero history); long decoding; greedy generation through the generation
entry point; the trace runner."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import pizitar_oracle as O

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

LA = dict(type="latent_attention", heads=3, dim=24, vdim=16, kv_rank=40, q_rank=20, ff=72)
LB = dict(type="latent_attention_2", heads=2, dim=16, vdim=24, kv_rank=72, ff=56)
MODELS = {
    # mixed stack: both mixers, a layer attending another's latents, a layer without feed-forward
    "mixed": dict(layers=[LA, LB, dict(LA, kv_from=0, heads=2, dim=8, vdim=8, q_rank=12, ff=None), dict(LB, scale=0.7)],
                  width=48, vocab=67, taps=3),
    # sizes that are no multiple of 8 (every product on the fp32 FMA tiles), one head, five taps, no soft cap
    "odd": dict(layers=[dict(LB, heads=1, dim=20, vdim=12, kv_rank=36, ff=50), dict(LA, heads=5, dim=12, vdim=20, kv_rank=68, q_rank=28, ff=None)],
                width=44, vocab=61, taps=5, softcap=None),
    # values a model may happen to make equal or 1
    "ones": dict(layers=[dict(LA, heads=1, dim=32, vdim=32, kv_rank=32, q_rank=32, ff=64), dict(LB, heads=4, dim=16, vdim=16, kv_rank=64, ff=64)],
                 width=64, vocab=64, taps=1),
    # a latent above 256 components (the attention kernel's shorter key tiles) and above 64 / 128 (more accumulators per lane)
    "wide_latent": dict(layers=[dict(LB, heads=2, dim=16, vdim=16, kv_rank=264, ff=None), dict(LA, heads=2, dim=16, vdim=8, kv_rank=136, q_rank=16, ff=32)],
                        width=32, vocab=40, taps=2),
}


def make(name, arith="f32", seed=0, gain=1.0, t_max=512, n_seq=1):
    from ming_univision_amd.configuration import PizitarConfig
    from ming_univision_amd.pizitar import PizitarDecoder
    cfg = O.random_config(**MODELS[name])
    sd = O.random_weights(cfg, seed, gain)
    dec = PizitarDecoder(PizitarConfig.from_dict(cfg), {k: v.cuda() for k, v in sd.items()}, t_max=t_max, n_seq=n_seq, arith=arith)
    return cfg, sd, dec


def toks(cfg, n, seed=1):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def err(got, want):
    want = want.double()
    return float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-9))


def run_portions(dec, seq, tokens, cuts):
    """Feed `tokens` to cache sequence `seq` in portions of the given sizes; returns the logits of every position."""
    out, at = [], 0
    for n in cuts:
        ids = torch.tensor(tokens[at:at + n], device="cuda")
        out.append(dec.logits(dec.forward_spans(dec.embed(ids), [(seq, n, at)])))
        at += n
    assert at == len(tokens)
    return torch.cat(out, 0)


# ---- operators alone -------------------------------------------------------------------------------------------------------
def _bf(t):
    return t.to(torch.bfloat16)


def test_norm_operators():
    from ming_univision_amd._lib import check, current_stream, lib, ptr
    g = torch.Generator().manual_seed(0)
    for M, n, eps in ((1, 44, 1e-5), (7, 192, 1e-6), (33, 1000, 1e-3)):
        x = torch.randn(M, n, generator=g) * 3 + 0.5
        w, b = _bf(1 + 0.3 * torch.randn(n, generator=g)), _bf(0.2 * torch.randn(n, generator=g))
        xd, wd, bd = x.cuda(), w.cuda(), b.cuda()              # named: a temporary's memory would be handed to the next one
        y = torch.empty_like(xd)
        y16 = torch.empty(M, n, dtype=torch.bfloat16, device="cuda")
        check(lib().mn_affine_ln_rows(ptr(xd), n, ptr(wd), ptr(bd), eps, ptr(y), n, ptr(y16), n, M, n, current_stream()))
        ref = O.affine_layer_norm(x.double(), w.double(), b.double(), eps)
        assert err(y, ref) < 1e-5 and err(y16.float(), ref) < 1e-2
        # gate * y -> norm -> residual add
        gpre, sub = torch.randn(M, n, generator=g), torch.randn(M, n, generator=g) * 2
        res, gd, sd_ = xd.clone(), gpre.cuda(), sub.cuda()
        check(lib().mn_gated_ln_residual(ptr(res), n, ptr(gd), n, ptr(sd_), n, ptr(wd), ptr(bd), eps, M, n,
                                         current_stream()))
        ref = x.double() + O.affine_layer_norm(torch.sigmoid(gpre.double()) * sub.double(), w.double(), b.double(), eps)
        assert err(res, ref) < 1e-5
        # unit-norm polynomial
        coef = _bf(torch.tensor([0.7, -0.4, 0.25, 0.1]))
        cd = coef.cuda()
        check(lib().mn_polynorm_rows(ptr(xd), n, ptr(cd), eps, ptr(y), n, None, 0, M, n, current_stream()))
        assert err(y, O.poly_norm(x.double(), coef.double(), eps)) < 1e-5
        # RMS norm scattered into an arena [n_seq = 3, t_max = M + 2, n]
        arena = torch.zeros(3, M + 2, n, device="cuda")
        seq = torch.full((M,), 2, dtype=torch.int32, device="cuda")
        slot = torch.arange(1, M + 1, dtype=torch.int32, device="cuda")
        check(lib().mn_rms_rows(ptr(xd), n, ptr(wd), eps, ptr(arena), n, None, 0, ptr(seq), ptr(slot), M + 2, M, n, current_stream()))
        ref = O.rms_norm(x.double(), w.double(), eps)
        assert err(arena[2, 1:M + 1], ref) < 1e-5 and float(arena[:2].abs().max()) == 0 and float(arena[2, 0].abs().max()) == 0


def test_tap_filter_with_state():
    """Two sequences, fed in three calls of different cuts (one row, several, a cut inside the filter's reach)."""
    from ming_univision_amd._lib import check, current_stream, lib, ptr
    from ming_univision_amd.sequences import rows_of_spans
    g = torch.Generator().manual_seed(1)
    n = 70
    for taps in (1, 2, 4, 6):
        w = _bf(torch.randn(n, taps, generator=g))
        wd = w.cuda()
        xs = {0: torch.randn(9, n, generator=g), 2: torch.randn(7, n, generator=g)}
        refs = {s: x.double() + O.causal_tap_filter(x.double(), w.double()) for s, x in xs.items()}
        state = torch.full((3, max(taps - 1, 1), n), 7.0, device="cuda")       # stale contents must not show
        at = {0: 0, 2: 0}
        for cut in ({0: 1, 2: 3}, {2: 2, 0: 6}, {0: 2, 2: 2}):
            spans = [(s, c, at[s]) for s, c in cut.items()]
            t = {k: (torch.from_numpy(v).cuda() if k != "max_len" else v) for k, v in rows_of_spans(spans, 4).items()}
            x = torch.cat([xs[s][at[s]:at[s] + c] for s, c in cut.items()]).cuda()
            y = torch.empty_like(x)
            M = x.shape[0]
            check(lib().mn_tap_filter_rows(ptr(x), n, ptr(wd), taps, ptr(state), ptr(t["row_seq"]), ptr(t["row_slot"]), ptr(t["row_back"]),
                                           ptr(y), n, None, 0, M, n, current_stream()))
            check(lib().mn_tap_state_update(ptr(x), n, taps, ptr(state), ptr(t["row_seq"]), ptr(t["row_back"]), M, n, current_stream()))
            r0 = 0
            for s, c in cut.items():
                assert err(y[r0:r0 + c], refs[s][at[s]:at[s] + c]) < 1e-6, (taps, cut, s)
                r0 += c
                at[s] += c


def test_fused_decode_rows():
    """The one-launch form of a sublayer boundary for rows that are alone in their sequences (gate / norm / residual of the last
    sublayer, the next input norm, the tap filter with its state) against the oracle's functions, fed row by row."""
    from ming_univision_amd._lib import check, current_stream, lib, ptr
    g = torch.Generator().manual_seed(3)
    for n, taps, eps in ((44, 1, 1e-5), (192, 4, 1e-6), (1000, 3, 1e-5), (4090, 2, 1e-6), (300, 8, 1e-5)):
        wa, ba, wb, bb = (_bf(1 + 0.3 * torch.randn(n, generator=g)) for _ in range(4))
        tw = _bf(torch.randn(n, taps, generator=g))
        steps, seqs = 6, [2, 0]                                      # two sequences, one row each per call
        x0 = torch.randn(len(seqs), n, generator=g)
        gs, ys = torch.randn(steps, len(seqs), n, generator=g), torch.randn(steps, len(seqs), n, generator=g)
        dev = [t.cuda() for t in (wa, ba, wb, bb, tw)]
        state = torch.full((3, max(taps - 1, 1), n), 5.0, device="cuda")
        row_seq = torch.tensor(seqs, dtype=torch.int32, device="cuda")
        x = x0.cuda()
        xr, hist = x0.double().clone(), [[] for _ in seqs]
        for t in range(steps):
            slot = torch.full((len(seqs),), t, dtype=torch.int32, device="cuda")
            gd, yd = gs[t].cuda(), ys[t].cuda()
            nout, h = torch.empty_like(x), torch.empty_like(x)
            gated = t % 2 == 1                                       # with and without the first stage
            check(lib().mn_gated_norm_filter_rows(ptr(x), n, ptr(gd) if gated else None, n, ptr(yd), n, ptr(dev[0]), ptr(dev[1]), ptr(dev[2]),
                                                  ptr(dev[3]), eps, ptr(nout), n, ptr(dev[4]), taps, ptr(state), ptr(row_seq), ptr(slot),
                                                  ptr(h), n, len(seqs), n, current_stream()))
            if gated:
                xr = xr + O.affine_layer_norm(torch.sigmoid(gs[t].double()) * ys[t].double(), wa.double(), ba.double(), eps)
            nr = O.affine_layer_norm(xr, wb.double(), bb.double(), eps)
            assert err(x, xr) < 1e-5 and err(nout, nr) < 1e-5, (n, t)
            for k in range(len(seqs)):
                hist[k].append(nr[k])
                seqn = torch.stack(hist[k])
                want = (seqn + O.causal_tap_filter(seqn, tw.double()))[-1]
                assert err(h[k], want) < 1e-5, (n, taps, t, k)


def test_fp32_batched_product():
    from ming_univision_amd._lib import check, current_stream, lib, ptr
    g = torch.Generator().manual_seed(2)
    for M, N, K, B in ((1, 40, 24, 3), (5, 7, 3, 1), (16, 64, 16, 2), (17, 65, 17, 2), (33, 70, 130, 3), (64, 9, 40, 1), (65, 66, 20, 2), (200, 130, 72, 5)):
        a = torch.randn(M, B * K, generator=g)
        w = _bf(torch.randn(B, N, K, generator=g))
        bias = _bf(torch.randn(N, generator=g))
        gate = torch.randn(M, B * N, generator=g)
        c = torch.empty(M, B * N, device="cuda")
        c16 = torch.empty(M, B * N, dtype=torch.bfloat16, device="cuda")
        ad, wd, bd, gd = a.cuda(), w.cuda(), bias.cuda(), gate.cuda()
        check(lib().mn_gemm_f32_batched(ptr(ad), B * K, K, ptr(wd), K, N * K, ptr(bd), ptr(c), B * N, N, ptr(c16), B * N, N,
                                        ptr(gd), B * N, N, M, N, K, B, 0.37, current_stream()))
        ref = torch.cat([(0.37 * a[:, z * K:(z + 1) * K].double() @ w[z].double().T + bias.double()) *
                         torch.sigmoid(gate[:, z * N:(z + 1) * N].double()) for z in range(B)], 1)
        assert err(c, ref) < 1e-5 and err(c16.float(), ref) < 1e-2


VARIANTS = {"mfma": 0, "valu": 1}


def _attend(q, arena, seq, lens, H, r, block_rows, ks, variant="mfma"):
    """mn_latent_attn_ex (fp32 matrix-core kernel or the plain one) on rows that are consecutive positions of ONE sequence."""
    from ming_univision_amd._lib import check, current_stream, lib, ptr
    M = q.shape[0]
    row_seq = torch.full((M,), seq, dtype=torch.int32, device="cuda")
    row_len = torch.tensor(lens, dtype=torch.int32, device="cuda")
    b0 = np.arange(0, M, block_rows)
    blk = torch.tensor(np.stack([b0, np.minimum(block_rows, M - b0)], 1), dtype=torch.int32, device="cuda").contiguous()
    lat = torch.empty(M, H, r, device="cuda")
    nb = lib().mn_latent_attn_workspace_bytes(M, H, r, ks)
    ws = torch.empty(max(nb, 16), dtype=torch.uint8, device="cuda")
    check(lib().mn_latent_attn_ex(ptr(q), ptr(arena), ptr(row_seq), ptr(row_len), ptr(blk), blk.shape[0], M, H, r, arena.shape[1], max(lens), ks,
                                  ptr(lat), ptr(ws), ws.numel(), VARIANTS[variant], current_stream()))
    return lat


@pytest.mark.parametrize("variant", list(VARIANTS))
@pytest.mark.parametrize("r,H", [(40, 3), (64, 5), (72, 1), (136, 2), (264, 2), (520, 1), (48, 20)])
def test_latent_attention_needles(r, H, variant):
    """One key is made to dominate (the query is a large multiple of that key's latent): the result is that latent if and only if
    the key is inside the row's length.  Needles at the first slot, around the kernel's key-tile edges (16 / 32 / 64 keys), around the
    edges of forced key splits, and at the row's last visible slot; the same query with the length one shorter must not see it."""
    from ming_univision_amd._lib import lib
    g = torch.Generator().manual_seed(r)
    T, br = 300, lib().mn_latent_attn_block_rows()
    arena = torch.randn(2, T, r, generator=g)
    ad = arena.cuda()
    for ks in (1, 3):
        for needle in (0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 95, 96, 127, 128, 191, 192, 255, 256, 298, 299):
            c = arena[1, needle].double()
            q1 = (40.0 / float(c @ c)) * c                                  # score 40 at the needle, |score| ~ 40 / sqrt(r) elsewhere
            q = torch.stack([torch.stack([q1.float() * (1 + 0.01 * h) for h in range(H)])] * 2)         # two rows, same query
            lat = _attend(q.cuda(), ad, 1, [needle, needle + 1] if needle else [1, 1], H, r, br, ks, variant)
            ref = []
            for ln in ([needle, needle + 1] if needle else [1, 1]):
                p = torch.softmax(arena[1, :ln].double() @ q[0].double().T, 0)                         # [ln, H]
                ref.append(p.T @ arena[1, :ln].double())
            ref = torch.stack(ref)
            assert err(lat, ref) < 2e-5, (ks, needle)
            assert float((lat[1, 0].cpu().double() - c).abs().max()) < 1e-2 * float(c.abs().max()), (ks, needle)
            if needle:
                assert float((lat[0, 0].cpu().double() - c).abs().max()) > 0.1 * float(c.abs().max()), (ks, needle)


@pytest.mark.parametrize("variant", list(VARIANTS))
def test_latent_attention_against_expanded_heads(variant):
    """Absorbed attention (queries mapped into latent space, values expanded afterwards) = attention on per-head keys and values."""
    g = torch.Generator().manual_seed(5)
    H, d, v, r, T = 3, 24, 16, 40, 150
    c = torch.randn(T, r, generator=g)
    q = torch.randn(T, H * d, generator=g)
    uk, uv = _bf(torch.randn(H * d, r, generator=g) * 0.3), _bf(torch.randn(H * v, r, generator=g) * 0.3)
    ref = O.latent_attention_core(q.double(), c.double(), uk.double(), uv.double(), H, d, v, 0.2)
    qabs = torch.stack([0.2 * q[:, h * d:(h + 1) * d].double() @ uk[h * d:(h + 1) * d].double() for h in range(H)], 1).float()
    arena = torch.zeros(1, T + 5, r)
    arena[0, :T] = c
    for block_rows, ks in ((4, 1), (1, 2), (3, 4)):
        lat = _attend(qabs.cuda(), arena.cuda(), 0, list(range(1, T + 1)), H, r, block_rows, ks, variant).cpu().double()
        out = torch.cat([lat[:, h] @ uv[h * v:(h + 1) * v].double().T for h in range(H)], 1)
        assert err(out, ref) < 1e-5


# ---- whole models ------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", list(MODELS))
def test_prompt_layers_and_logits(name):
    cfg, sd, dec = make(name)
    t = toks(cfg, 90)
    trace = []
    ref = O.logits_of(cfg, sd, t, trace=trace)
    hid, tr = dec.forward_spans(dec.embed(torch.tensor(t, device="cuda")), [(0, len(t), 0)], trace=True)
    for i, want in enumerate(trace):
        assert err(tr[i], want) < 1e-4, f"residual stream after layer {i}"
    assert err(dec.logits(hid), ref) < 1e-4


@pytest.mark.parametrize("name", ["mixed", "odd", "ones"])
def test_first_tokens(name):
    """Prompts of 1, 2, 3 tokens, and a sequence decoded from its very first token on (the filter's history starts empty)."""
    cfg, sd, dec = make(name)
    for n in (1, 2, 3):
        t = toks(cfg, n, seed=10 + n)
        assert err(run_portions(dec, 0, t, [n]), O.logits_of(cfg, sd, t)) < 1e-4
    t = toks(cfg, 9, seed=3)
    assert err(run_portions(dec, 0, t, [1] * 9), O.logits_of(cfg, sd, t)) < 1e-4


@pytest.mark.parametrize("name", ["mixed", "odd", "wide_latent"])
def test_portions_and_decoding(name):
    """Prompt in one portion / in portions of changing size down to two tokens / token by token: each equals the oracle (and
    therefore each other); the decoding runs across the attention kernel's 64-key tile edge and a portion cut falls inside the
    filter's reach of the previous portion."""
    cfg, sd, dec = make(name)
    t = toks(cfg, 140)
    ref = O.logits_of(cfg, sd, t)
    for cuts in ([140], [37, 2, 3, 2, 60, 1, 1, 2, 32], [50] + [1] * 90, [2] * 70):
        assert err(run_portions(dec, 0, t, cuts), ref) < 1e-4, cuts


def test_unequal_requests_share_a_pass():
    """Three requests of different lengths in one pass, then a pass that mixes a prompt portion of one with single decode rows of
    the others: every request's logits equal the oracle on that request alone."""
    cfg, sd, dec = make("mixed", n_seq=4)
    reqs = {3: toks(cfg, 70, 1), 0: toks(cfg, 9, 2), 2: toks(cfg, 33, 3)}
    refs = {s: O.logits_of(cfg, sd, t) for s, t in reqs.items()}
    first = {3: 40, 0: 8, 2: 32}
    ids = torch.tensor([x for s, t in reqs.items() for x in t[:first[s]]], device="cuda")
    lg = dec.logits(dec.forward_spans(dec.embed(ids), [(s, first[s], 0) for s in reqs]))
    r0 = 0
    for s in reqs:
        assert err(lg[r0:r0 + first[s]], refs[s][:first[s]]) < 1e-4
        r0 += first[s]
    ids = torch.tensor([reqs[0][8]] + reqs[3][40:70] + [reqs[2][32]], device="cuda")
    lg = dec.logits(dec.forward_spans(dec.embed(ids), [(0, 1, 8), (3, 30, 40), (2, 1, 32)]))
    assert err(lg[0:1], refs[0][8:9]) < 1e-4 and err(lg[1:31], refs[3][40:70]) < 1e-4 and err(lg[31:32], refs[2][32:33]) < 1e-4


def test_inputs_longer_than_a_pass(monkeypatch):
    """More rows than one pass through the stack takes: the passes cut a sequence in the middle (inside the filter's reach and
    inside a key tile) and a later sequence starts inside a pass; the per-layer trace is stitched across passes."""
    from ming_univision_amd import pizitar
    monkeypatch.setattr(pizitar, "MAX_ROWS", 37)
    cfg, sd, dec = make("mixed", n_seq=2)
    a, b = toks(cfg, 90, 1), toks(cfg, 50, 2)
    trace = []
    ra, rb = O.logits_of(cfg, sd, a, trace=trace), O.logits_of(cfg, sd, b)
    ids = torch.tensor(a + b, device="cuda")
    hid, tr = dec.forward_spans(dec.embed(ids), [(1, 90, 0), (0, 50, 0)], trace=True)
    lg = dec.logits(hid)
    assert err(lg[:90], ra) < 1e-4 and err(lg[90:], rb) < 1e-4
    assert err(tr[-1][:90], trace[-1]) < 1e-4
    with pytest.raises(AssertionError):
        dec.forward_spans(dec.embed(ids[:10]), [(0, 10, dec.t_max - 5)])       # beyond the arena: refused, not written


def test_released_sequences_are_reused():
    """A cache sequence that held a longer request is given back and reused: the old latents and filter state stay in memory and
    must not leak into the next request (nothing is cleared; lengths bound every read)."""
    from ming_univision_amd.sequences import SequenceSlots
    cfg, sd, dec = make("mixed")
    slots = SequenceSlots(dec)
    a, b = slots.alloc(), slots.alloc()
    assert (a, b) == (0, 1) and dec.n_seq >= 2
    long_, other = toks(cfg, 100, 1), toks(cfg, 20, 2)
    run_portions(dec, a, long_, [100])
    run_portions(dec, b, other, [20])
    slots.release(a)
    assert slots.alloc() == a
    t = toks(cfg, 30, 4)
    assert err(run_portions(dec, a, t, [3, 1, 1, 25]), O.logits_of(cfg, sd, t)) < 1e-4
    c = slots.alloc()                                     # growing the arenas keeps live sequences
    assert c == 2 and dec.n_seq >= 3
    more = toks(cfg, 6, 6)
    got = dec.logits(dec.forward_spans(dec.embed(torch.tensor(more, device="cuda")), [(a, 6, 30)]))
    assert err(got, O.logits_of(cfg, sd, t + more)[30:]) < 1e-4


def test_far_key_decides_the_logits():
    """Peaky attention (scores scaled up), so single far keys carry the result: a prompt of 260 tokens, its last 40 decoded one by
    one.  A key lost anywhere (first slot, a tile's edge, the newest slot) shows in the logits."""
    cfg, sd, dec = make("mixed", gain=3.0, seed=7)
    t = toks(cfg, 260, 9)
    ref = O.logits_of(cfg, sd, t)
    assert err(run_portions(dec, 0, t, [220] + [1] * 40), ref) < 2e-4


def test_long_decoding():
    cfg, sd, dec = make("odd")
    t = toks(cfg, 330, 11)
    got = run_portions(dec, 0, t, [5] + [1] * 325)
    assert err(got, O.logits_of(cfg, sd, t)) < 1e-4


def test_bf16_arithmetic():
    """Serving arithmetic: portions above 64 rows take the bf16 MFMA products (3e-2 of the logits' scale against the oracle),
    portions of 9 .. 64 rows the weight-streaming MFMA route on hi/lo rows, rows fed a few at a time fp32 FMA."""
    for name in ("ones", "mixed"):                      # "mixed": some products have a K that is no multiple of 8 and stay on fp32 FMA
        cfg, sd, dec = make(name, arith="bf16")
        t = toks(cfg, 150)
        ref = O.logits_of(cfg, sd, t)
        assert err(run_portions(dec, 0, t, [150]), ref) < 3e-2                   # tiled MFMA GEMM (above 64 rows)
        assert err(run_portions(dec, 0, t, [70, 40, 31, 9]), ref) < 3e-2         # + the weight-streaming MFMA route (9 .. 64 rows)
        assert err(run_portions(dec, 0, t[:40], [1] * 40), ref[:40]) < 1e-4      # fp32 FMA
        assert err(run_portions(dec, 0, t[:64], [12, 20, 32]), ref[:64]) < 5e-3  # hi/lo rows (measured 2e-3; the tiled GEMM 6e-3 .. 9e-3)


def test_greedy_generation_entry_point():
    """PizitarForCausalLM.generate: unequal prompts in one lock-step batch; every new token is the oracle's arg-max given the
    tokens before it (or the oracle's two best are within 1e-4), alone or batched; sampled generation returns tokens and gives its
    cache sequences back."""
    from ming_univision_amd.pizitar import PizitarForCausalLM
    cfg, sd, dec = make("mixed")
    lm = PizitarForCausalLM(dec)
    prompts = [toks(cfg, 17, 1), toks(cfg, 3, 2), toks(cfg, 66, 3)]
    new = lm.generate(prompts, max_new_tokens=12)
    alone = [lm.generate([p], max_new_tokens=12)[0] for p in prompts]
    for p, out, solo in zip(prompts, new, alone):
        assert len(out) == 12
        ref = O.logits_of(cfg, sd, p + out)
        for i, tok in enumerate(out):
            row = ref[len(p) - 1 + i]
            top = torch.topk(row, 2).values
            assert int(row.argmax()) == tok or float(top[0] - row[tok]) < 1e-4
        assert solo == out
    assert not lm.slots.length and lm.slots.next == 3
    out = lm.generate(prompts, max_new_tokens=5, do_sample=True, top_k=8, generator=torch.Generator(device="cuda").manual_seed(0))
    assert all(len(o) == 5 and all(0 <= x < cfg["vocab"] for x in o) for o in out) and not lm.slots.length


def test_decode_graph_replays():
    """The captured decode step against the eager one: every replay is checked (not only the first), with eager work and host
    synchronisations between replays, across a re-capture (the lengths pass the captured bound) and the 16-key tile edges."""
    cfg, sd, dec = make("mixed", n_seq=3)
    prompts = {0: toks(cfg, 21, 1), 1: toks(cfg, 5, 2), 2: toks(cfg, 40, 3)}
    follow = {s: toks(cfg, 30, 10 + s) for s in prompts}
    refs = {s: O.logits_of(cfg, sd, prompts[s] + follow[s]) for s in prompts}
    for s, p in prompts.items():
        run_portions(dec, s, p, [len(p)])
    row_seq = torch.tensor(list(prompts), dtype=torch.int32, device="cuda")
    slot = torch.tensor([len(p) for p in prompts.values()], dtype=torch.int32, device="cuda")
    ln = slot + 1
    g = dec.decode_graph(row_seq, slot, ln)
    g.span = 16                                               # re-capture every 16 tokens
    other = dec.embed(torch.tensor(toks(cfg, 7, 99), device="cuda"))
    for i in range(30):
        ids = torch.tensor([follow[s][i] for s in prompts], device="cuda")
        hid = g.run(dec.embed(ids), max(len(p) for p in prompts.values()) + i + 1)
        lg = dec.logits(hid.clone())
        torch.cuda.synchronize()
        for k, s in enumerate(prompts):
            assert err(lg[k:k + 1], refs[s][len(prompts[s]) + i][None]) < 1e-4, (i, s)
        dec.logits(other)                                     # eager work between replays
    assert slot.tolist() == [len(p) + 30 for p in prompts.values()]
    from ming_univision_amd.pizitar import PizitarForCausalLM
    lm = PizitarForCausalLM(dec)
    ps = [toks(cfg, 9, 5), toks(cfg, 30, 6)]
    assert lm.generate(ps, max_new_tokens=20, use_graph=True) == lm.generate(ps, max_new_tokens=20, use_graph=False)


def test_trace_runner(tmp_path):
    """bin/trace_run on a saved model: a request in portions interleaved with a second one, logits against the oracle; the first
    request's cache sequence is reused by a third."""
    from safetensors.torch import save_file
    cfg = O.random_config(**MODELS["mixed"])
    sd = O.random_weights(cfg, 3)
    mdir, odir = tmp_path / "model", tmp_path / "out"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(mdir / "model.safetensors"))
    a, b, c = toks(cfg, 25, 1), toks(cfg, 6, 2), toks(cfg, 11, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:10], "want": [0, 9]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:5], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[10:12], "want": [1]}, {"id": "b", "tokens": b[5:], "want": [0]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[12:], "want": [12]}], "end": ["a"]},
        {"step": 4, "entries": [{"id": "c", "tokens": c, "want": [0, 10]}], "end": ["c"]},
    ]
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 3e-2)):
        r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dtype, "--out", str(odir), "--max-tokens", "64"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(5)]
        ra, rb, rc = (O.logits_of(cfg, sd, x) for x in (a, b, c))
        want = {0: ra[[0, 9]], 2: torch.stack([ra[11], rb[5]]), 3: ra[[24]], 4: rc[[0, 10]]}
        assert not (odir / "1.f32").exists()
        for n, ref in want.items():
            got = torch.from_numpy(np.fromfile(odir / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]))
            assert err(got, ref) < tol, (dtype, n)
            os.unlink(odir / f"{n}.f32")
