"""Host-side pieces of the Sakinex integration that need no GPU: configuration reading and validation, the registry's choice by
config.json, parameter shapes, the order of layer runs, and the oracle's own consistency (what a position sees; the equivalence of
its position-by-position attention with a dense masked softmax; the recurrence in closed form)."""
import copy
import json

import pytest
import torch

from ming_univision_amd.configuration import SakinexConfig, config_from_pretrained, sakinex_param_shapes
from tests import sakinex_oracle as O


def test_config_and_registry(tmp_path):
    cfg = O.small_config(no_mlp=(2,))
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    name, c = config_from_pretrained(str(tmp_path))
    assert name == "sakinex" and isinstance(c, SakinexConfig)
    assert (c.width, c.vocab, c.taps, c.eps, c.residual_mult) == (64, 96, 3, 1e-5, 0.7)
    sh = sakinex_param_shapes(c)
    assert sh == O.tensor_shapes(cfg)
    assert "l2.mlp.router" not in sh and "l2.norm2" not in sh and "l2.canon2" not in sh and sh["l0.mix.left.k"] == (32, 64)
    assert sh["l1.mix.left.o"] == (64, 96) and sh["l0.mlp.shared.sg"] == (1, 64) and sh["l0.mix.left.v.conv"] == (48, 3)
    bare = copy.deepcopy(cfg)
    bare.pop("canon"), bare.pop("loop")
    for k in ("conv", "rot", "mask"):
        bare["layers"][0]["mixer"]["left"].pop(k)
    bare["layers"][0]["mlp"].pop("shared")
    c2 = SakinexConfig.from_dict(bare)
    sh2 = sakinex_param_shapes(c2)
    assert sh2 == O.tensor_shapes(bare) and c2.taps == 0 and "l0.canon1" not in sh2 and "l0.mix.left.q.conv" not in sh2
    assert "l0.mlp.shared.gate" not in sh2 and "l1.mlp.shared.gate" in sh2


@pytest.mark.parametrize("loop,want", [
    (None, [0, 1, 2, 3]), ((0, 3, 2), [0, 1, 2, 0, 1, 2, 3]), ((1, 2, 2), [0, 1, 1, 2, 3]), ((2, 4, 2), [0, 1, 2, 3, 2, 3]),
    ((0, 4, 1), [0, 1, 2, 3]), ((3, 3, 5), [0, 1, 2, 3])])
def test_order_of_layer_runs(loop, want):
    cfg = O.small_config(n_layers=4, loop=loop)
    c = SakinexConfig.from_dict(cfg)
    assert [i for i, _ in c.runs()] == want == [i for i, _ in O.layer_runs(cfg)]
    assert c.runs() == O.layer_runs(cfg)
    if loop and loop[2] > 1 and loop[1] > loop[0]:
        again = [k for k, (_, a) in enumerate(c.runs()) if a]
        assert len(again) == loop[2] - 1 and all(c.runs()[k][0] == loop[0] for k in again)
    else:
        assert not any(a for _, a in c.runs())


@pytest.mark.parametrize("edit", [
    lambda c: c["layers"][0].update(type="serial"), lambda c: c["layers"][0]["mixer"]["left"].pop("scale"),
    lambda c: c["layers"][0]["mixer"]["left"].update(heads=3), lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7),
    lambda c: c["layers"][1]["mlp"].update(kind="dense"), lambda c: c["layers"][1]["mlp"]["router"].update(top=9),
    lambda c: c.update(loop=dict(start=2, stop=1, times=2)), lambda c: c["layers"][0]["mixer"].pop("right_scale")])
def test_config_validation(edit):
    cfg = copy.deepcopy(O.small_config())
    edit(cfg)
    with pytest.raises(ValueError):
        SakinexConfig.from_dict(cfg)


def test_what_a_position_sees():
    mask = {"size": 5, "pool": 3}
    assert O.visible(0, mask) == ([0], [])
    assert O.visible(4, mask) == ([0, 1, 2, 3, 4], [])
    assert O.visible(6, mask) == ([2, 3, 4, 5, 6], [])           # tokens 0 and 1 have left the window, their block is not whole outside it
    assert O.visible(7, mask) == ([3, 4, 5, 6, 7], [0])          # block 0 = tokens 0 .. 2 lies wholly before the window
    assert O.visible(9, mask) == ([5, 6, 7, 8, 9], [0])
    assert O.visible(10, mask) == ([6, 7, 8, 9, 10], [0, 1])
    assert O.visible(6, {"size": 5}) == ([2, 3, 4, 5, 6], [])
    assert O.visible(6, None) == (list(range(7)), [])


def test_attention_equals_a_dense_masked_softmax():
    g = torch.Generator().manual_seed(0)
    T, H, G, d, e, S, P = 23, 4, 2, 6, 5, 5, 3
    q, k, v = (torch.randn(T, n, c, generator=g, dtype=torch.float64) for n, c in ((H, d), (G, d), (G, e)))
    got = O.windowed_attention(q, k, v, 0.8, {"size": S, "pool": P})
    nb = T // P
    kk = torch.cat([k[:nb * P].reshape(nb, P, G, d).mean(1), k])          # block means, then tokens
    vv = torch.cat([v[:nb * P].reshape(nb, P, G, e).mean(1), v])
    i = torch.arange(T)[:, None]
    see_tok = (i - torch.arange(T)[None] >= 0) & (i - torch.arange(T)[None] < S)
    see_blk = (torch.arange(nb)[None] * P + P - 1) <= i - S
    see = torch.cat([see_blk, see_tok], 1)
    for h in range(H):
        s = (q[:, h] @ kk[:, h // 2].T) * 0.8
        p = torch.softmax(s.masked_fill(~see, float("-inf")), -1)
        assert torch.allclose(p @ vv[:, h // 2], got[:, h], atol=1e-12)


def test_recurrence_in_closed_form():
    g = torch.Generator().manual_seed(1)
    T, W, n = 9, 7, 5
    sd = {"z": torch.randn(n, W, generator=g), "z.b": torch.randn(n, generator=g), "x": torch.randn(n, W, generator=g),
          "x.b": torch.randn(n, generator=g), "g": torch.randn(n, W, generator=g), "o": torch.eye(n)}
    sd = {k: v.double() for k, v in sd.items()}
    h = torch.randn(T, W, generator=g, dtype=torch.float64)
    out = O.min_gru(h, sd, "")
    z, c = torch.sigmoid(h @ sd["z"].T + sd["z.b"]), O.gru_candidate(h @ sd["x"].T + sd["x.b"])
    S = sum(z[s] * c[s] * torch.prod(1 - z[s + 1:T], 0) for s in range(T))     # S_T = sum_s z_s c_s prod_(r > s) (1 - z_r)
    gate = h[-1] @ sd["g"].T
    assert torch.allclose(out[-1], S * gate * torch.sigmoid(gate), atol=1e-12)
    u = torch.tensor([-2.0, -1e-9, 0.0, 3.0], dtype=torch.float64)
    assert torch.allclose(O.gru_candidate(u), torch.tensor([1 / (1 + 2.718281828459045 ** 2), 0.5, 0.5, 3.5], dtype=torch.float64), atol=1e-9)


def test_rotary_frequencies_ramp():
    rot = {"base": 100.0, "dims": 8, "scaling": {"factor": 4.0, "fast": 8.0, "original": 16, "slow": 1.0}}
    f, mag = O.rotary_frequencies(rot)
    plain, one = O.rotary_frequencies({"base": 100.0, "dims": 8})
    assert one == 1.0 and abs(mag - (0.1 * 1.3862943611198906 + 1)) < 1e-12
    assert torch.all(f <= plain + 1e-15) and torch.all(f >= plain / 4 - 1e-15)
    assert f[0] == plain[0]                                       # the fastest pair keeps its frequency
    x = torch.randn(3, 2, 12, dtype=torch.float64)
    y = O.rotate(x, torch.tensor([0, 5, 9]), rot)
    assert torch.equal(y[..., 8:], x[..., 8:]) and torch.allclose(y[0], x[0] * torch.cat([torch.full((8,), mag), torch.ones(4)]).double())
