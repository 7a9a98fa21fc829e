"""Sakinex on the HIP path against tests/sakinex_oracle.py (plain float64 restatement, one function per mechanism).

Small random models of several shapes (sizes that are no multiples of 8, one head, as many key/value heads as query heads, more
than 8 query heads per key/value head, one tap, blocks of one token, a window longer than the sequence, no window at all, every
expert chosen, more experts than the sorted route takes, layers without feed-forward, repeated ranges at the start / middle / not at
all).  fp32 arithmetic is held to 1e-4 of the logits' scale, the bf16-MFMA arithmetic to 3e-2.  Covers: every operator alone;
whole prompts with the residual stream after every layer run; token-by-token decoding; portions down to two tokens; several
unequal requests in one pass against each alone; cache sequences that are released and reused; keys just inside and just outside
the window, blocks that are just seen and not yet seen, in prompts and in decoding, with scores scaled up so that one key decides;
the first positions of a sequence; long decoding; greedy generation through the generation entry point; the captured decode
step; the trace runner."""
import copy
import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

from tests import sakinex_oracle as O

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

MODELS = {
    # repeated middle layer, grouped key/value heads, rotation on part of a head, a layer without feed-forward
    "mixed": dict(no_mlp=(2,)),
    # sizes that are no multiple of 8 (every product on the fp32 FMA kernels), every expert chosen, five taps, plain frequencies
    "odd": dict(width=44, vocab=61, n_layers=2, heads=3, kv_heads=1, dim=10, vdim=18, rot_dims=6, conv=2, window=7, pool=3, gru=36, experts=3,
                top=3, ff=50, shared_ff=10, taps=5, loop=None, scaling=False, mult=0.5),
    # values a model may happen to make equal or 1
    "ones": dict(width=32, vocab=32, n_layers=2, heads=2, kv_heads=2, dim=16, vdim=16, rot_dims=16, conv=1, window=1, pool=1, gru=32, experts=2,
                 top=1, ff=32, shared_ff=32, taps=1, loop=(0, 2, 1), mult=1.0),
    # twelve query heads on one key/value head (two chunks of the attention launch), a window longer than any test sequence, more
    # experts than the sorted route takes, the repeated range at the start
    # layers that differ from each other in every size (edited in config()), a repeated range of two layers at the end
    "varied": dict(width=72, vocab=50, n_layers=4, loop=(2, 4, 2), no_mlp=(3,)),
    "wide": dict(width=32, vocab=40, n_layers=2, heads=12, kv_heads=1, dim=8, vdim=8, rot_dims=4, window=500, pool=16, gru=24, experts=130,
                 top=4, ff=8, shared_ff=8, loop=(0, 1, 3)),
}


def config(name):
    cfg = O.small_config(**MODELS[name])
    if name == "varied":                                 # no two layers alike: every size, window, filter and router differs
        cfg = copy.deepcopy(cfg)
        a, b = cfg["layers"][1], cfg["layers"][2]
        a["mixer"]["left"].update(heads=2, kv_heads=1, dim=24, vdim=8, conv=2, scale=0.2, mask={"size": 5, "pool": 2},
                                  rot={"base": 1000.0, "dims": 24})
        a["mixer"].update(left_scale=1.1, right_scale=0.3, right={"width": 24})
        a["mlp"].update(router={"experts": 3, "top": 1}, expert={"ff": 40}, shared={"ff": 72})
        b["mixer"]["left"].update(heads=6, kv_heads=6, dim=8, vdim=40, conv=5, mask={"size": 33})
        b["mixer"].update(right={"width": 100})
        b["mlp"].update(router={"experts": 9, "top": 4}, expert={"ff": 16})
        b["mlp"].pop("shared")
    if name == "wide":                                   # optional keys left out: no filters, no window, no rotation, no shared expert
        cfg = copy.deepcopy(cfg)
        ly = cfg["layers"][1]
        for k in ("conv", "mask", "rot"):
            ly["mixer"]["left"].pop(k)
        ly["mlp"].pop("shared")
    return cfg


def build(cfg, sd, arith="f32", t_max=512, n_seq=1):
    from ming_univision_amd.configuration import SakinexConfig
    from ming_univision_amd.sakinex import SakinexDecoder
    return SakinexDecoder(SakinexConfig.from_dict(cfg), {k: v.cuda() for k, v in sd.items()}, t_max=t_max, n_seq=n_seq, arith=arith)


def make(name, arith="f32", seed=0, t_max=512, n_seq=1, peaky=1.0):
    cfg = config(name)
    if peaky != 1.0:
        cfg = copy.deepcopy(cfg)
        for ly in cfg["layers"]:
            ly["mixer"]["left"]["scale"] *= peaky
    sd = O.random_weights(cfg, seed)
    return cfg, sd, build(cfg, sd, arith, t_max, n_seq)


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


def _api():
    from ming_univision_amd._lib import check, current_stream, lib, ptr
    return check, current_stream, lib(), ptr


def _rows(spans):
    from ming_univision_amd.sequences import rows_of_spans
    t = rows_of_spans(spans, 1 << 30)
    return {k: torch.from_numpy(v).cuda() for k, v in t.items() if k != "max_len"}


def _bf(t):
    return t.to(torch.bfloat16)


_KEEP = []


def D(t):
    """A device copy that outlives the launch it is passed to (the pointer alone would not keep the memory)."""
    _KEEP.append(t.cuda())
    return _KEEP[-1]


@pytest.fixture(autouse=True)
def _drop_device_copies():
    yield
    torch.cuda.synchronize()
    _KEEP.clear()


# ---- operators alone -------------------------------------------------------------------------------------------------------
def test_residual_norm_rows_and_fused_decode_rows():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(0)
    for M, n, taps, eps in ((1, 44, 3, 1e-5), (5, 256, 1, 1e-6), (9, 1000, 8, 1e-3), (3, 300, 2, 1e-6), (2, 2048, 4, 1e-6), (4, 1028, 4, 1e-6),
                            (2, 250, 4, 1e-6), (3, 64, 1, 1e-6), (2, 520, 6, 1e-6)):
        x, y = torch.randn(M, n, generator=g) * 2, torch.randn(M, n, generator=g)
        w, tw = _bf(1 + 0.2 * torch.randn(n, generator=g)), _bf(0.5 * torch.randn(n, taps, generator=g))
        state = torch.randn(4, max(taps - 1, 1), n, generator=g)
        xs = x.double() + 0.7 * y.double()
        nref = O.rms_norm(xs, w.double(), eps)
        xd, nd, n16 = x.cuda(), torch.empty(M, n, device="cuda"), torch.empty(M, n, dtype=torch.bfloat16, device="cuda")
        check(L.mn_axpy_rms_rows(ptr(xd), n, ptr(D(y)), n, 0.7, ptr(D(w)), eps, ptr(nd), n, ptr(n16), n, M, n, stream()))
        assert err(xd, xs) < 1e-6 and err(nd, nref) < 1e-5 and err(n16.float(), nref) < 1e-2
        # decode rows: row r is position slot[r] of sequence seq[r]; entry i of its state is its input i + 1 positions back
        seq = torch.tensor([(3 * r + 1) % 4 for r in range(M)][:M], dtype=torch.int32)
        if M > 4:
            continue                                      # distinct rows need distinct sequences
        slot = torch.tensor([0, 1, 5, 9][:M], dtype=torch.int32)
        href = nref.clone()
        for r in range(M):
            hist = [nref[r]] + [state[seq[r], i].double() if slot[r] - (i + 1) >= 0 else torch.zeros(n, dtype=torch.float64) for i in range(taps - 1)]
            for k in range(taps):
                href[r] += tw[:, taps - 1 - k].double() * hist[k]
        xd, hd, sdev = x.cuda(), torch.empty(M, n, device="cuda"), state.cuda()
        check(L.mn_axpy_rms_filter_rows(ptr(xd), n, ptr(D(y)), n, 0.7, ptr(D(w)), eps, ptr(D(tw)), taps, ptr(sdev), ptr(D(seq)),
                                        ptr(D(slot)), ptr(hd), n, M, n, stream()))
        assert err(xd, xs) < 1e-6 and err(hd, href) < 1e-5
        for r in range(M):
            if taps > 1:
                assert err(sdev[seq[r], 0], nref[r]) < 1e-5
            for i in range(1, taps - 1):
                assert torch.equal(sdev[seq[r], i].cpu(), state[seq[r], i - 1])


def test_channel_filter_without_the_input():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(1)
    n, taps, ld = 70, 4, 90
    u = torch.randn(23, ld, generator=g)
    w = _bf(torch.randn(n, taps, generator=g))
    ref = O.causal_taps(u[:, :n].double(), w.double())
    state = torch.zeros(2, taps - 1, n, device="cuda")
    got, at = [], 0
    for cut in (5, 1, 2, 15):
        r = _rows([(1, cut, at)])
        y = torch.empty(cut, n, device="cuda")
        xs = u[at:at + cut].cuda()
        check(L.mn_tap_conv_rows(ptr(xs), ld, ptr(D(w)), taps, ptr(state), ptr(r["row_seq"]), ptr(r["row_slot"]), ptr(r["row_back"]), ptr(y), n,
                                 cut, n, stream()))
        check(L.mn_tap_state_update(ptr(xs), ld, taps, ptr(state), ptr(r["row_seq"]), ptr(r["row_back"]), cut, n, stream()))
        got.append(y)
        at += cut
    assert err(torch.cat(got), ref) < 1e-6


@pytest.mark.parametrize("H,G,dim,vdim,rot", [
    (4, 2, 16, 24, dict(base=100.0, dims=8, scaling=dict(factor=4.0, fast=8.0, original=16, slow=1.0))),
    (3, 1, 12, 20, dict(base=10000.0, dims=12)), (2, 2, 40, 8, None),
    (1, 1, 136, 8, dict(base=500000.0, dims=130, scaling=dict(factor=32.0, fast=32.0, original=8192, slow=1.0)))])
def test_rotation_unit_norm_and_append(H, G, dim, vdim, rot):
    from ming_univision_amd.sakinex import rotary_table
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(2)
    M, t_max, eps, scale = 6, 5000, 1e-5, 0.37
    pos = torch.tensor([0, 1, 2, 77, 1500, 4999])
    qkv = torch.randn(M, (H + G) * dim + G * vdim, generator=g)
    q, k, v = qkv[:, :H * dim].double().reshape(M, H, dim), qkv[:, H * dim:(H + G) * dim].double().reshape(M, G, dim), qkv[:, (H + G) * dim:]
    qref, kref = O.rms_unit(O.rotate(q, pos, rot), eps) * scale, O.rms_unit(O.rotate(k, pos, rot), eps)
    freq, mag, dims = None, 1.0, 0
    if rot:
        freq, mag = rotary_table(rot, "cuda")
        dims = rot["dims"]
        fref, mref = O.rotary_frequencies(rot)
        assert err(freq, fref) < 1e-7 and abs(mag - mref) < 1e-6
    seq = torch.tensor([1, 0, 1, 0, 1, 0], dtype=torch.int32).cuda()
    slot = pos.to(torch.int32).cuda()
    qo = torch.empty(M, H * dim, device="cuda")
    ka, va = torch.zeros(2, t_max, G * dim, device="cuda"), torch.zeros(2, t_max, G * vdim, device="cuda")
    check(L.mn_rope_unit_append(ptr(D(qkv)), qkv.shape[1], M, H, G, dim, vdim, dims, ptr(freq), mag, 1, eps, scale, ptr(seq), ptr(slot),
                                ptr(qo), H * dim, ptr(ka), ptr(va), t_max, stream()))
    assert err(qo, qref.reshape(M, -1)) < 1e-4                     # fp32 frequencies and angles at position 4999: 3e-5
    for m in range(M):
        assert err(ka[seq[m], pos[m]], kref[m].reshape(-1)) < 1e-4
        assert torch.equal(va[seq[m], pos[m]].cpu(), v[m])
    assert int((ka != 0).any(-1).sum()) == M


@pytest.mark.parametrize("H,G,dim,vdim,conv,pool,dims", [(4, 2, 16, 24, 3, 4, 8), (3, 1, 12, 20, 2, 3, 6), (2, 2, 16, 16, 1, 1, 16), (2, 1, 8, 8, 0, 0, 0),
                                                         (1, 1, 136, 8, 5, 2, 130)])
def test_decode_rows_filter_rotation_append_and_block_means_in_one_launch(H, G, dim, vdim, conv, pool, dims):
    """The fused launch of decode rows against the chain of operators it stands for (channel filter, its state update, rotation and
    append, block means), on rows of four sequences at positions that do and do not complete a block and have less history than taps."""
    from ming_univision_amd.sakinex import rotary_table
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(11)
    C, t_max, M, n_seq = (H + G) * dim + G * vdim, 40, 4, 5
    npm = t_max // max(pool, 1) + 1
    freq, mag = rotary_table(dict(base=50.0, dims=dims, scaling=dict(factor=4.0, fast=8.0, original=16, slow=1.0)), "cuda") if dims else (None, 1.0)
    pin = torch.randn(M, C + 7, generator=g).cuda()
    w = _bf(torch.randn(C, max(conv, 1), generator=g)).cuda()
    seq = torch.tensor([3, 0, 4, 1], dtype=torch.int32).cuda()
    slot = torch.tensor([0, 1, 2 * max(pool, 1) - 1 + 8, 11], dtype=torch.int32).cuda()
    back = torch.zeros(M, dtype=torch.int32).cuda()
    init = dict(state=torch.randn(n_seq, max(conv - 1, 1), C, generator=g), ka=torch.randn(n_seq, t_max, G * dim, generator=g),
                va=torch.randn(n_seq, t_max, G * vdim, generator=g), pk=torch.randn(n_seq, npm, G * dim, generator=g),
                pv=torch.randn(n_seq, npm, G * vdim, generator=g))
    a = {k: v.cuda() for k, v in init.items()}
    b = {k: v.cuda() for k, v in init.items()}
    qa, qb, tmp = torch.empty(M, H * dim, device="cuda"), torch.empty(M, H * dim, device="cuda"), torch.empty(M, C, device="cuda")
    ng = 300
    zx, gg = torch.randn(M, 2 * ng + 1, generator=g).cuda(), torch.randn(M, ng, generator=g).cuda()
    gst = torch.randn(n_seq, ng, generator=g)
    gst_a, gst_b, go_a, go_b = gst.cuda(), gst.cuda(), torch.zeros(M, ng + 3, device="cuda"), torch.zeros(M, ng + 3, device="cuda")
    src, ld = pin, C + 7
    if conv:
        check(L.mn_tap_conv_rows(ptr(pin), C + 7, ptr(w), conv, ptr(a["state"]), ptr(seq), ptr(slot), ptr(back), ptr(tmp), C, M, C, stream()))
        check(L.mn_tap_state_update(ptr(pin), C + 7, conv, ptr(a["state"]), ptr(seq), ptr(back), M, C, stream()))
        src, ld = tmp, C
    check(L.mn_rope_unit_append(ptr(src), ld, M, H, G, dim, vdim, dims, ptr(freq), mag, 1, 1e-6, 0.3, ptr(seq), ptr(slot), ptr(qa), H * dim, ptr(a["ka"]),
                                ptr(a["va"]), t_max, stream()))
    if pool:
        check(L.mn_pool_blocks_update(ptr(a["ka"]), ptr(a["va"]), t_max, ptr(a["pk"]), ptr(a["pv"]), npm, pool, G * dim, G * vdim, ptr(seq), ptr(slot), M,
                                      stream()))
    check(L.mn_filter_rope_append_rows(ptr(pin), C + 7, M, H, G, dim, vdim, ptr(w) if conv else None, conv, ptr(b["state"]), dims, ptr(freq), mag, 1, 1e-6,
                                       0.3, ptr(seq), ptr(slot), ptr(qb), H * dim, ptr(b["ka"]), ptr(b["va"]), t_max, ptr(b["pk"]) if pool else None,
                                       ptr(b["pv"]) if pool else None, npm, pool, ptr(zx), 2 * ng + 1, ptr(gg), ng, ptr(gst_b), ng, 0.4, ptr(go_b), ng + 3,
                                       stream()))
    check(L.mn_mingru_rows(ptr(zx), 2 * ng + 1, ptr(gg), ng, ptr(gst_a), ptr(seq), ptr(slot), ptr(back), 0.4, ptr(go_a), ng + 3, None, 0, M, ng,
                           stream()))
    assert err(go_b[:, :ng], go_a[:, :ng].cpu()) < 1e-6 and err(gst_b, gst_a.cpu()) < 1e-6      # the recurrence of the same rows rides the launch
    assert err(qb, qa.cpu()) < 1e-6
    for k in a:
        assert err(b[k], a[k].cpu()) < 1e-6, k
    assert pool == 0 or not torch.equal(a["pk"].cpu(), init["pk"])          # some row did complete a block
    assert conv <= 1 or not torch.equal(a["state"].cpu(), init["state"])


def _attention_case(T, H, G, dim, vdim, window, pool, peaky, seed, rows=None):
    """Random unit-norm keys in an arena, the block means by the framework's own kernel, attention of `rows` (default all) against
    the oracle's."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(seed)
    q = O.rms_unit(torch.randn(T, H, dim, generator=g).double(), 0.0) * peaky / math.sqrt(dim)
    k, v = O.rms_unit(torch.randn(T, G, dim, generator=g).double(), 0.0), torch.randn(T, G, vdim, generator=g).double()
    mask = None if window == 0 else ({"size": window, "pool": pool} if pool else {"size": window})
    ref = O.windowed_attention(q, k, v, 1.0, mask, rows).reshape(T, H * vdim)
    t_max, npm = T + 3, (T // pool + 1 if pool else 1)
    ka, va = torch.zeros(2, t_max, G * dim, device="cuda"), torch.zeros(2, t_max, G * vdim, device="cuda")
    ka[1, :T], va[1, :T] = k.reshape(T, -1).float().cuda(), v.reshape(T, -1).float().cuda()
    pk, pv = torch.full((2, npm, G * dim), float("nan"), device="cuda"), torch.full((2, npm, G * vdim), float("nan"), device="cuda")
    r = _rows([(1, T, 0)])
    if pool:
        check(L.mn_pool_blocks_update(ptr(ka), ptr(va), t_max, ptr(pk), ptr(pv), npm, pool, G * dim, G * vdim, ptr(r["row_seq"]), ptr(r["row_slot"]), T,
                                      stream()))
        nb = T // pool
        assert err(pk[1, :nb], k[:nb * pool].reshape(nb, pool, -1).mean(1)) < 1e-6
    rows = list(range(T)) if rows is None else rows
    sel = torch.tensor(rows)
    qd = q.reshape(T, -1).float()[sel].cuda()
    out = torch.empty(len(rows), H * vdim + 5, device="cuda")
    out16 = torch.empty(len(rows), H * vdim, dtype=torch.bfloat16, device="cuda")
    rs, rp = r["row_seq"][sel.cuda()].contiguous(), r["row_slot"][sel.cuda()].contiguous()     # held until the results are read
    check(L.mn_window_pool_attn(ptr(qd), H * dim, ptr(ka), ptr(va), ptr(pk) if pool else None, ptr(pv) if pool else None, ptr(rs), ptr(rp),
                                len(rows), H, G, dim, vdim, t_max, npm, window, pool, 0.6, ptr(out), H * vdim + 5, ptr(out16), H * vdim, stream()))
    assert err(out[:, :H * vdim], 0.6 * ref[sel]) < 2e-5
    assert err(out16.float(), 0.6 * ref[sel]) < 1e-2
    # the tiled form: single rows with several key splits, then runs of up to block_rows consecutive rows
    from ming_univision_amd.sequences import rows_of_spans
    for nsplit in (1, 3, 64):
        out.fill_(float("nan"))
        ws = torch.empty(max(16, L.mn_window_attn_workspace_bytes(len(rows), H, G, vdim, 1, nsplit)), dtype=torch.uint8, device="cuda")
        check(L.mn_window_pool_attn_blocks(ptr(qd), H * dim, ptr(ka), ptr(va), ptr(pk) if pool else None, ptr(pv) if pool else None, ptr(rs), ptr(rp),
                                           None, len(rows), 1, H, G, dim, vdim, t_max, npm, window, pool, 0.6, ptr(out), H * vdim + 5, ptr(out16),
                                           H * vdim, nsplit, ptr(ws), ws.numel(), stream()))
        assert err(out[:, :H * vdim], 0.6 * ref[sel]) < 2e-5, nsplit
        assert err(out16.float(), 0.6 * ref[sel]) < 1e-2
    if len(rows) == T:
        RB = L.mn_window_attn_block_rows()
        for past in (0, 3):                                   # runs that start at position 0, and runs that straddle block and window edges otherwise
            spans = [(1, past, 0), (1, T - past, past)] if past else [(1, T, 0)]
            tb = rows_of_spans(spans, RB)
            blk = torch.from_numpy(tb["blk_tab"]).cuda()
            for nsplit, variant in ((1, 0), (2, 0), (5, 0), (1, 1), (2, 1)):          # 0: fp32 matrix cores, 1: fp32 FMA
                if variant == 0 and max(dim, vdim) > 256:
                    continue
                outb = torch.full((T, H * vdim), float("nan"), device="cuda")
                ob16 = torch.empty(T, H * vdim, dtype=torch.bfloat16, device="cuda")
                ws = torch.empty(max(16, L.mn_window_attn_workspace_bytes(blk.shape[0], H, G, vdim, 0, nsplit)), dtype=torch.uint8, device="cuda")
                check(L.mn_window_pool_attn_blocks_ex(ptr(qd), H * dim, ptr(ka), ptr(va), ptr(pk) if pool else None, ptr(pv) if pool else None,
                                                      ptr(r["row_seq"]), ptr(r["row_slot"]), ptr(blk), blk.shape[0], 0, H, G, dim, vdim, t_max, npm,
                                                      window, pool, 0.6, ptr(outb), H * vdim, ptr(ob16), H * vdim, nsplit, ptr(ws), ws.numel(), variant,
                                                      stream()))
                assert err(outb, 0.6 * ref) < 2e-5, (past, nsplit, variant)
                assert err(ob16.float(), 0.6 * ref) < 1e-2


@pytest.mark.parametrize("H,G,dim,vdim,window,pool", [(4, 2, 16, 24, 9, 4), (3, 1, 12, 20, 7, 3), (2, 2, 16, 16, 1, 1), (12, 1, 8, 8, 0, 0),
                                                      (1, 1, 40, 72, 16, 0), (9, 1, 20, 12, 5, 8), (2, 1, 136, 264, 4, 2), (3, 1, 18, 10, 6, 3), (5, 5, 7, 3, 11, 2)])
def test_window_and_pooled_blocks_one_key_decides(H, G, dim, vdim, window, pool):
    """Scores scaled up until the softmax is nearly a pick of one key: a token kept one position too long, dropped one too early,
    or a block seen one position early changes whole rows."""
    _attention_case(70, H, G, dim, vdim, window, pool, peaky=40.0, seed=3)
    _attention_case(70, H, G, dim, vdim, window, pool, peaky=3.0, seed=4)


def test_attention_over_several_key_tiles():
    """More than 256 visible keys: block means and window tokens on both sides of a tile's edge; a window cut by the sequence's start."""
    _attention_case(900, 2, 1, 16, 16, 300, 2, peaky=30.0, seed=5, rows=[0, 1, 254, 255, 256, 257, 299, 300, 301, 511, 512, 513, 555, 811, 812, 899])
    _attention_case(600, 3, 1, 8, 8, 0, 0, peaky=30.0, seed=6, rows=[0, 255, 256, 257, 511, 512, 599])
    _attention_case(200, 8, 2, 72, 136, 37, 5, peaky=30.0, seed=7)       # every row, in runs: heads of 72 / 136 values (padded 64-blocks)
    _attention_case(150, 2, 2, 200, 40, 0, 0, peaky=20.0, seed=8)        # one query head per key/value head, no window


def test_min_gru_rows_carry_their_state():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(7)
    n, T = 70, 40
    zx, gg = torch.randn(T, 2 * n + 3, generator=g) * 2, torch.randn(T, n, generator=g)
    z, c = torch.sigmoid(zx[:, :n].double()), O.gru_candidate(zx[:, n:2 * n].double())
    S, ref = torch.zeros(n, dtype=torch.float64), []
    for t in range(T):
        S = (1 - z[t]) * S + z[t] * c[t]
        ref.append(0.5 * S * gg[t].double() * torch.sigmoid(gg[t].double()))
    ref = torch.stack(ref)
    state = torch.full((3, n), 7.0, device="cuda")              # a reused slot: whatever it holds, position 0 starts from zero
    got, at = [], 0
    for cut in (6, 1, 1, 2, 30):
        r = _rows([(2, cut, at)])
        out = torch.empty(cut, n, device="cuda")
        check(L.mn_mingru_rows(ptr(D(zx[at:at + cut])), zx.shape[1], ptr(D(gg[at:at + cut])), n, ptr(state), ptr(r["row_seq"]), ptr(r["row_slot"]),
                               ptr(r["row_back"]), 0.5, ptr(out), n, None, 0, cut, n, stream()))
        got.append(out)
        at += cut
    assert err(torch.cat(got), ref) < 1e-5 and err(state[2], S) < 1e-5 and float(state[0].min()) == 7.0
    # two sequences in one call
    r = _rows([(0, 4, 0), (1, 3, 0)])
    out = torch.empty(7, n, device="cuda")
    check(L.mn_mingru_rows(ptr(D(torch.cat([zx[:4], zx[:3]]))), zx.shape[1], ptr(D(torch.cat([gg[:4], gg[:3]]))), n, ptr(state), ptr(r["row_seq"]),
                           ptr(r["row_slot"]), ptr(r["row_back"]), 0.5, ptr(out), n, None, 0, 7, n, stream()))
    assert err(out[:4], ref[:4]) < 1e-5 and err(out[4:], ref[:3]) < 1e-5
    # the chunked scan: a sequence that continues from its state, one that starts, one of a single row, chunk edges inside them
    zx2, gg2 = torch.randn(150, 2 * n + 3, generator=g) * 2, torch.randn(150, n, generator=g)
    st0 = torch.randn(4, n, generator=g)
    spans = [(3, 70, 5), (0, 1, 0), (1, 47, 0), (2, 32, 9)]
    want, fin, at = [], {}, 0
    for seq, cnt, past in spans:
        S = st0[seq].double() if past else torch.zeros(n, dtype=torch.float64)
        for t in range(at, at + cnt):
            z, c = torch.sigmoid(zx2[t, :n].double()), O.gru_candidate(zx2[t, n:2 * n].double())
            S = (1 - z) * S + z * c
            want.append(0.5 * S * gg2[t].double() * torch.sigmoid(gg2[t].double()))
        fin[seq], at = S, at + cnt
    r = _rows(spans)
    for scan in (True, False):
        std, out = st0.cuda(), torch.empty(150, n + 2, device="cuda")
        o16 = torch.empty(150, n, dtype=torch.bfloat16, device="cuda")
        if scan:
            ws = torch.empty(L.mn_mingru_scan_workspace_bytes(150, n), dtype=torch.uint8, device="cuda")
            check(L.mn_mingru_rows_scan(ptr(D(zx2)), zx2.shape[1], ptr(D(gg2)), n, ptr(std), ptr(r["row_seq"]), ptr(r["row_slot"]), ptr(r["row_back"]), 0.5,
                                        ptr(out), n + 2, ptr(o16), n, 150, n, ptr(ws), ws.numel(), stream()))
        else:
            check(L.mn_mingru_rows(ptr(D(zx2)), zx2.shape[1], ptr(D(gg2)), n, ptr(std), ptr(r["row_seq"]), ptr(r["row_slot"]), ptr(r["row_back"]), 0.5,
                                   ptr(out), n + 2, ptr(o16), n, 150, n, stream()))
        assert err(out[:, :n], torch.stack(want)) < 1e-5 and err(o16.float(), torch.stack(want)) < 1e-2, scan
        for seq in fin:
            assert err(std[seq], fin[seq]) < 1e-5, (scan, seq)


def test_router_and_expert_operators():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(8)
    for M, E, top in ((5, 10, 3), (3, 130, 4), (2, 3, 3), (4, 2, 1), (1, 700, 9)):
        z = torch.randn(M, E + 2, generator=g)
        z[0, 1] = z[0, 0] = z[0, :E].max() + 1                      # a tie at the top: the lower index first
        val, idx = torch.topk(z[:, :E].double(), top, dim=-1)
        wref = torch.softmax(val, -1)
        di, dw = torch.empty(M, top, dtype=torch.int32, device="cuda"), torch.empty(M, top, device="cuda")
        check(L.mn_router_topk_rows(ptr(D(z)), E + 2, M, E, top, ptr(di), ptr(dw), stream()))
        assert di[0, :2].tolist() == [0, 1][:top]
        assert torch.equal(di[1:].cpu().long(), idx[1:]) and err(dw, wref) < 1e-6
    M, n, K, E, top = 4, 37, 52, 5, 2
    x = torch.randn(M, 2 * n, generator=g)
    y = torch.empty(M, n, device="cuda")
    check(L.mn_silu_mul_rows(ptr(D(x)), 2 * n, ptr(y), n, None, 0, M, n, stream()))
    assert err(y, torch.nn.functional.silu(x[:, :n].double()) * x[:, n:].double()) < 1e-6
    for M2, n2 in ((1, 300), (5, 37), (3, 700)):                   # the router's pick and the shared activation of few rows in one launch
        z, x2 = torch.randn(M2, 9, generator=g), torch.randn(M2, 2 * n2 + 2, generator=g)
        val, idx = torch.topk(z[:, :7].double(), 3, dim=-1)
        di, dw, y2 = torch.empty(M2, 3, dtype=torch.int32, device="cuda"), torch.empty(M2, 3, device="cuda"), torch.zeros(M2, n2 + 1, device="cuda")
        check(L.mn_router_topk_silu_rows(ptr(D(z)), 9, M2, 7, 3, ptr(di), ptr(dw), ptr(D(x2)), 2 * n2 + 2, ptr(y2), n2 + 1, n2, stream()))
        assert torch.equal(di.cpu().long(), idx) and err(dw, torch.softmax(val, -1)) < 1e-6
        assert err(y2[:, :n2], torch.nn.functional.silu(x2[:, :n2].double()) * x2[:, n2:2 * n2].double()) < 1e-6 and float(y2[:, n2].abs().max()) == 0.0
    for K_ in (K, 64):                                              # scalar and 8-wide weight loads
        a, w = torch.randn(M, K_, generator=g), _bf(torch.randn(E, n, K_, generator=g))
        idx = torch.randint(0, E, (M * top,), generator=g).to(torch.int32)
        c = torch.empty(M * top, n, device="cuda")
        check(L.mn_gemv_f32_indexed(ptr(D(a)), K_, top, ptr(D(w)), K_, n * K_, ptr(D(idx)), ptr(c), n, M * top, n, K_, stream()))
        ref = torch.stack([w[idx[zz]].double() @ a[zz // top].double() for zz in range(M * top)])
        assert err(c, ref) < 1e-5
    xr, ye, sh, sg, tw = (torch.randn(s, generator=g) for s in ((M, n), (M * top, n), (M, n), (M, 3), (M, top)))
    slot_of = torch.randperm(M * top, generator=g).to(torch.int32)
    for so in (None, slot_of):
        rows = ye if so is None else ye[so.long()]
        ref = xr.double() + 0.7 * ((tw.double()[:, :, None] * rows.double().reshape(M, top, n)).sum(1) + torch.sigmoid(sg[:, 1:2].double()) * sh.double())
        xd = xr.cuda()
        check(L.mn_moe_combine_residual(ptr(xd), n, ptr(D(ye)), n, ptr(D(so)) if so is not None else None, ptr(D(tw)), top, ptr(D(sh)), n,
                                        ptr(D(sg)[:, 1:]), 3, 0.7, M, n, stream()))
        assert err(xd, ref) < 1e-6


# ---- whole models ------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", list(MODELS))
def test_prompt_layers_and_logits(name):
    cfg, sd, dec = make(name)
    t = toks(cfg, 81)                                     # above 64 rows: the recurrence runs as a chunked scan
    ref, streams = O.forward(cfg, sd, t, trace=True)
    hid, tr = dec.forward_spans(dec.embed(torch.tensor(t, device="cuda")), [(0, len(t), 0)], trace=True)
    assert tr.shape[0] == len(O.layer_runs(cfg))
    for r in range(tr.shape[0]):
        assert err(tr[r], streams[r]) < 1e-4, r
    assert err(dec.logits(hid), ref) < 1e-4


@pytest.mark.parametrize("name", ["mixed", "odd", "ones"])
def test_first_tokens(name):
    """The first positions: zero history of both filters, a recurrence from zero, a window that is not full, no block yet."""
    cfg, sd, dec = make(name)
    t = toks(cfg, 6, 5)
    ref = O.forward(cfg, sd, t)
    assert err(run_portions(dec, 0, t, [1] * 6), ref) < 1e-4
    assert err(run_portions(dec, 0, t, [2, 2, 2]), ref) < 1e-4
    assert err(run_portions(dec, 0, t[:1], [1]), ref[:1]) < 1e-4


@pytest.mark.parametrize("name", list(MODELS))
def test_portions_and_decoding(name):
    cfg, sd, dec = make(name)
    t = toks(cfg, 75, 2)
    ref = O.forward(cfg, sd, t)
    assert err(run_portions(dec, 0, t, [40] + [1] * 35), ref) < 1e-4                       # prefill against token-by-token decoding
    assert err(run_portions(dec, 0, t, [7, 2, 13, 2, 2, 1, 19, 3, 2, 24]), ref) < 1e-4     # portions cut inside windows and blocks
    assert err(run_portions(dec, 0, t, [1] * 75), ref) < 1e-4


def test_window_and_block_edges_in_prompts_and_decoding():
    """Peaky attention, so that single keys carry the result: a key just inside or outside the window and a block that is just
    seen or not yet change the logits of the positions around them, in portions and decoded one by one."""
    cfg, sd, dec = make("mixed", peaky=12.0, seed=7)
    t = toks(cfg, 64, 9)
    ref = O.forward(cfg, sd, t)
    assert err(run_portions(dec, 0, t, [64]), ref) < 2e-4
    assert err(run_portions(dec, 0, t, [8] + [1] * 56), ref) < 2e-4
    assert err(run_portions(dec, 0, t, [9, 3, 4, 5, 11, 2, 30]), ref) < 2e-4


def test_unequal_requests_share_a_pass():
    """Three requests of different lengths in one pass, then a pass that mixes a prompt portion of one with single decode rows of
    the others: every request's logits equal the oracle on that request alone."""
    cfg, sd, dec = make("mixed", n_seq=4)
    reqs = {3: toks(cfg, 50, 1), 0: toks(cfg, 9, 2), 2: toks(cfg, 33, 3)}
    refs = {s: O.forward(cfg, sd, t) for s, t in reqs.items()}
    first = {3: 30, 0: 8, 2: 32}
    ids = torch.tensor([x for s, t in reqs.items() for x in t[:first[s]]], device="cuda")
    lg = dec.logits(dec.forward_spans(dec.embed(ids), [(s, first[s], 0) for s in reqs]))
    r0 = 0
    for s in reqs:
        assert err(lg[r0:r0 + first[s]], refs[s][:first[s]]) < 1e-4
        r0 += first[s]
    ids = torch.tensor([reqs[0][8]] + reqs[3][30:50] + [reqs[2][32]], device="cuda")
    lg = dec.logits(dec.forward_spans(dec.embed(ids), [(0, 1, 8), (3, 20, 30), (2, 1, 32)]))
    assert err(lg[0:1], refs[0][8:9]) < 1e-4 and err(lg[1:21], refs[3][30:50]) < 1e-4 and err(lg[21:22], refs[2][32:33]) < 1e-4


def test_inputs_longer_than_a_pass(monkeypatch):
    """More rows than one pass through the stack takes: the passes cut a sequence inside the filters' reach, a window and a block,
    and a later sequence starts inside a pass; the trace is stitched across passes."""
    from ming_univision_amd import seq_lm
    monkeypatch.setattr(seq_lm, "MAX_ROWS", 23)
    cfg, sd, dec = make("mixed", n_seq=2)
    a, b = toks(cfg, 60, 1), toks(cfg, 31, 2)
    (ra, sa), rb = O.forward(cfg, sd, a, trace=True), O.forward(cfg, sd, b)
    ids = torch.tensor(a + b, device="cuda")
    hid, tr = dec.forward_spans(dec.embed(ids), [(1, 60, 0), (0, 31, 0)], trace=True)
    lg = dec.logits(hid)
    assert err(lg[:60], ra) < 1e-4 and err(lg[60:], rb) < 1e-4 and err(tr[-1][:60], sa[-1]) < 1e-4
    with pytest.raises(AssertionError):
        dec.forward_spans(dec.embed(ids[:10]), [(0, 10, dec.t_max - 5)])       # beyond the cache: refused, not written


def test_released_sequences_are_reused():
    """A cache sequence that held a longer request is given back and reused: its old keys, block means, filter and recurrent states
    stay in memory and must not leak into the next request (nothing is cleared)."""
    from ming_univision_amd.sequences import SequenceSlots
    cfg, sd, dec = make("mixed")
    slots = SequenceSlots(dec)
    a, b = slots.alloc(), slots.alloc()
    assert (a, b) == (0, 1) and dec.n_seq >= 2
    long_, other = toks(cfg, 70, 1), toks(cfg, 20, 2)
    run_portions(dec, a, long_, [70])
    run_portions(dec, b, other, [20])
    slots.release(a)
    assert slots.alloc() == a
    t = toks(cfg, 30, 4)
    assert err(run_portions(dec, a, t, [3, 1, 1, 25]), O.forward(cfg, sd, t)) < 1e-4
    c = slots.alloc()                                     # growing the caches keeps live sequences
    assert c == 2 and dec.n_seq >= 3
    more = toks(cfg, 6, 6)
    got = dec.logits(dec.forward_spans(dec.embed(torch.tensor(more, device="cuda")), [(a, 6, 30)]))
    assert err(got, O.forward(cfg, sd, t + more)[30:]) < 1e-4
    got = dec.logits(dec.forward_spans(dec.embed(torch.tensor(other[:5], device="cuda")), [(b, 5, 0)]))     # b starts again on its old slots
    assert err(got, O.forward(cfg, sd, other[:5])) < 1e-4


def test_long_decoding():
    cfg, sd, dec = make("odd")
    t = toks(cfg, 200, 11)
    got = run_portions(dec, 0, t, [5] + [1] * 195)
    assert err(got, O.forward(cfg, sd, t)) < 1e-4


def rows_off(got, want, tol):
    """-> (rows whose error is above tol of the logits' scale, median row error).  bf16-rounded router inputs may flip a close call
    between two experts, which changes single rows by more than rounding does; such rows are counted, not averaged away."""
    want = want.double()
    e = (got.double().cpu() - want).abs().amax(-1) / want.abs().max()
    return int((e > tol).sum()), float(e.median())


def test_bf16_arithmetic():
    """Serving arithmetic: portions above 64 rows take the bf16 MFMA products and the experts sorted on the grouped MFMA GEMM (rows
    within 3e-2 of the logits' scale against the oracle, but for at most 8 in 100 whose routing was a close call (130 experts make many); median below 1e-2),
    portions of 9 .. 64 rows the weight-streaming MFMA route on hi/lo rows, rows fed a few at a time fp32 FMA."""
    for name in ("mixed", "odd", "wide", "varied"):       # "odd": no K is a multiple of 8, "wide": too many experts for the sorted route
        cfg, sd, dec = make(name, arith="bf16")
        t = toks(cfg, 100)
        ref = O.forward(cfg, sd, t)
        for cuts in ([100], [70, 21, 9]):
            off, med = rows_off(run_portions(dec, 0, t, cuts), ref, 3e-2)
            assert off <= 8 and med < 1e-2, (name, cuts, off, med)
        assert err(run_portions(dec, 0, t[:30], [1] * 30), ref[:30]) < 1e-4
        off, med = rows_off(run_portions(dec, 0, t[:64], [12, 20, 32]), ref[:64], 5e-3)
        assert off <= 5 and med < 2e-3, (name, off, med)


def test_greedy_generation_entry_point():
    """SakinexForCausalLM.generate: unequal prompts in one lock-step batch; every new token is the oracle's arg-max given the
    tokens before it (or the oracle's two best are within 1e-4), alone or batched, with and without the captured decode step;
    sampled generation returns tokens and gives its cache sequences back."""
    from ming_univision_amd.sakinex import SakinexForCausalLM
    cfg, sd, dec = make("mixed")
    lm = SakinexForCausalLM(dec)
    prompts = [toks(cfg, 17, 1), toks(cfg, 3, 2), toks(cfg, 40, 3)]
    new = lm.generate(prompts, max_new_tokens=12)
    alone = [lm.generate([p], max_new_tokens=12, use_graph=False)[0] for p in prompts]
    for p, out, solo in zip(prompts, new, alone):
        assert len(out) == 12
        ref = O.forward(cfg, sd, p + out)
        for i, tok in enumerate(out):
            row = ref[len(p) - 1 + i]
            top = torch.topk(row, 2).values
            assert int(row.argmax()) == tok or float(top[0] - row[tok]) < 1e-4
        assert solo == out
    assert not lm.slots.length and lm.slots.next == 3
    out = lm.generate(prompts, max_new_tokens=5, do_sample=True, top_k=8, generator=torch.Generator(device="cuda").manual_seed(0))
    assert all(len(o) == 5 and all(0 <= x < cfg["vocab"] for x in o) for o in out) and not lm.slots.length


def test_decode_graph_replays():
    """The captured decode step against the oracle: every replay is checked (not only the first), with eager work and host
    synchronisations between replays, across a re-capture, while windows slide and blocks complete."""
    cfg, sd, dec = make("mixed", n_seq=3)
    prompts = {0: toks(cfg, 21, 1), 1: toks(cfg, 5, 2), 2: toks(cfg, 30, 3)}
    follow = {s: toks(cfg, 24, 10 + s) for s in prompts}
    refs = {s: O.forward(cfg, sd, prompts[s] + follow[s]) for s in prompts}
    for s, p in prompts.items():
        run_portions(dec, s, p, [len(p)])
    row_seq = torch.tensor(list(prompts), dtype=torch.int32, device="cuda")
    slot = torch.tensor([len(p) for p in prompts.values()], dtype=torch.int32, device="cuda")
    ln = slot + 1
    g = dec.decode_graph(row_seq, slot, ln)
    g.span = 16                                               # re-capture every 16 tokens
    other = dec.embed(torch.tensor(toks(cfg, 7, 99), device="cuda"))
    for i in range(24):
        ids = torch.tensor([follow[s][i] for s in prompts], device="cuda")
        hid = g.run(dec.embed(ids), max(len(p) for p in prompts.values()) + i + 1)
        lg = dec.logits(hid.clone())
        torch.cuda.synchronize()
        for k, s in enumerate(prompts):
            assert err(lg[k:k + 1], refs[s][len(prompts[s]) + i][None]) < 1e-4, (i, s)
        dec.logits(other)                                     # eager work between replays
    assert slot.tolist() == [len(p) + 24 for p in prompts.values()]


def test_decode_batches_on_the_grouped_expert_route_replay_as_a_graph():
    """Ten sequences per decode step in the serving arithmetic: the experts run sorted on the grouped 256-tile MFMA GEMM (width and
    expert width multiples of 64).  The captured step, replayed, picks the same tokens as the eager one, and the logits of the batch
    stay within the bf16 tolerance of the oracle."""
    from ming_univision_amd.sakinex import SakinexForCausalLM
    cfg = O.small_config(width=64, ff=64, shared_ff=64, gru=64, experts=5, top=2, loop=(0, 1, 2), n_layers=2)
    sd = O.random_weights(cfg, 5)
    dec = build(cfg, sd, arith="bf16", t_max=128, n_seq=10)
    lm = SakinexForCausalLM(dec)
    prompts = [toks(cfg, 3 + 2 * i, 20 + i) for i in range(10)]
    a = lm.generate(prompts, max_new_tokens=12, use_graph=True)
    b = lm.generate(prompts, max_new_tokens=12, use_graph=False)
    assert a == b
    full = [p + o for p, o in zip(prompts, a)]
    ids = torch.tensor([t for f in full for t in f], device="cuda")
    lg = dec.logits(dec.forward_spans(dec.embed(ids), [(i, len(f), 0) for i, f in enumerate(full)]))
    r0, off = 0, 0
    for f in full:
        n_off, med = rows_off(lg[r0:r0 + len(f)], O.forward(cfg, sd, f), 3e-2)
        off, r0 = off + n_off, r0 + len(f)
        assert med < 1e-2
    assert off <= 8


def test_trace_runner(tmp_path):
    """bin/trace_run on a saved model: a request in portions interleaved with a second one, logits against the oracle; the first
    request's cache sequence is reused by a third."""
    from safetensors.torch import save_file
    cfg = config("mixed")
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
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 5e-2)):
        r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dtype, "--out", str(odir), "--max-tokens", "64"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(5)]
        ra, rb, rc = (O.forward(cfg, sd, x) for x in (a, b, c))
        want = {0: ra[[0, 9]], 2: torch.stack([ra[11], rb[5]]), 3: ra[[24]], 4: rc[[0, 10]]}
        assert not (odir / "1.f32").exists()
        for n, ref in want.items():
            got = torch.from_numpy(np.fromfile(odir / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]))
            assert err(got, ref) < tol, (dtype, n)
            os.unlink(odir / f"{n}.f32")
