"""Daberax without a GPU: configuration, registry and tensor shapes of the package, and the float64 restatement held against
independent closed forms (what a position sees, the frequency bands, the filter's causality, the delta rule as explicit sums)."""
import json
import math

import pytest
import torch

from ming_univision_amd.configuration import DaberaxConfig, config_from_pretrained, daberax_param_shapes
from tests import daberax_oracle as O


def small():
    return O.small_config([O.latent_layer(window=5, mlp=O.dense(24)), O.delta_layer(mlp=None),
                           O.attention_layer(softcap=3.0, window=7, scaling=(4.0, 1.0, 4.0, 64), mlp=O.dense(40))])


def test_config_registry_and_shapes(tmp_path):
    cfg = small()
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    name, c = config_from_pretrained(str(tmp_path))
    assert name == "daberax" and isinstance(c, DaberaxConfig) and c.side_dim == 6 and c.logit_scale == 0.5 and c.eps == 1e-5
    assert {k: tuple(v) for k, v in daberax_param_shapes(c).items()} == {k: tuple(v) for k, v in O.param_shapes(cfg).items()}
    assert "l1.norm2" not in daberax_param_shapes(c) and "l1.side.gate" in daberax_param_shapes(c)
    plain = DaberaxConfig.from_dict({**cfg, "token_side": None})
    assert plain.side_dim == 0 and "side.embed" not in daberax_param_shapes(plain)
    assert DaberaxConfig.from_dict(c.to_dict()).to_dict() == c.to_dict()


@pytest.mark.parametrize("edit, text", [
    (lambda c: c["layers"][0].update(type="conv"), "unknown mixer"),
    (lambda c: c["layers"][2]["mixer"].update(kv_heads=3), "do not divide"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=5), "even"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["layers"][1]["mixer"].pop("conv"), "lacks"),
    (lambda c: c["layers"][0].update(mlp={"kind": "moe", "ff": 8}), "feed-forward"),
])
def test_config_validation(edit, text):
    cfg = small()
    edit(cfg)
    with pytest.raises(ValueError, match=text):
        DaberaxConfig.from_dict(cfg)


def test_what_a_position_sees():
    m = O.visible(9, 3)
    for i in range(9):
        assert [j for j in range(9) if m[i, j]] == [j for j in range(9) if 0 <= i - j < 3]
    assert bool((O.visible(5, None) == torch.ones(5, 5, dtype=torch.bool).tril()).all())
    assert bool((O.visible(5, 1) == torch.eye(5, dtype=torch.bool)).all())


def test_frequency_bands():
    rot = {"base": 10000.0, "dims": 32, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 100}}
    f, plain = O.rotary_frequencies(rot), O.rotary_frequencies({"base": 10000.0, "dims": 32})
    for fi, pi in zip(f.tolist(), plain.tolist()):
        wave = 2 * math.pi / pi
        if wave < 25:
            assert fi == pi
        elif wave > 100:
            assert abs(fi - pi / 4) < 1e-15
        else:
            assert pi / 4 < fi < pi
    assert float(plain[0]) == 1.0 and abs(float(plain[1]) - 10000 ** (-2 / 32)) < 1e-15


def test_rotation_is_a_rotation_of_interleaved_pairs():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 3, 10, generator=g, dtype=torch.float64)
    f = torch.tensor([1.0, 0.3, 0.01], dtype=torch.float64)
    y = O.rotate_interleaved(x, f, pos0=5)
    assert bool((y[..., 6:] == x[..., 6:]).all())
    for t in range(7):
        for i in range(3):
            a = (5 + t) * float(f[i])
            assert torch.allclose(y[t, :, 2 * i], x[t, :, 2 * i] * math.cos(a) - x[t, :, 2 * i + 1] * math.sin(a))
            assert torch.allclose(y[t, :, 2 * i + 1], x[t, :, 2 * i + 1] * math.cos(a) + x[t, :, 2 * i] * math.sin(a))
    # scores depend on the distance only
    q, k = torch.randn(1, 1, 6, generator=g, dtype=torch.float64), torch.randn(1, 1, 6, generator=g, dtype=torch.float64)
    s1 = (O.rotate_interleaved(q, f, 9) * O.rotate_interleaved(k, f, 4)).sum()
    s2 = (O.rotate_interleaved(q, f, 105) * O.rotate_interleaved(k, f, 100)).sum()
    assert abs(float(s1 - s2)) < 1e-12


def test_filter_is_causal_and_ends_on_the_current_row():
    g = torch.Generator().manual_seed(1)
    x, w = torch.randn(8, 3, generator=g, dtype=torch.float64), torch.randn(3, 4, generator=g, dtype=torch.float64)
    y = O.causal_conv(x, w)
    for t in range(8):
        want = sum(w[:, 3 - k] * x[t - k] for k in range(4) if t - k >= 0)
        assert torch.allclose(y[t], want)
    x2 = x.clone()
    x2[5:] += 1.0
    assert bool((O.causal_conv(x2, w)[:5] == y[:5]).all())


def test_delta_rule_against_explicit_sums():
    """Without decay and with orthonormal keys a full-strength write replaces what its key held; with decay g and no overlap between
    keys the read-out is the sum of the writes, each faded by the decays since."""
    T, d, e = 6, 8, 3
    g = torch.Generator().manual_seed(2)
    k = torch.eye(d, dtype=torch.float64)[:T].reshape(T, 1, d)
    v = torch.randn(T, 1, e, generator=g, dtype=torch.float64)
    q = torch.randn(T, 1, d, generator=g, dtype=torch.float64)
    beta, dec = torch.rand(T, 1, generator=g, dtype=torch.float64), torch.rand(T, 1, generator=g, dtype=torch.float64)
    out, S = O.gated_delta_rule(q, k, v, beta, dec)
    for t in range(T):
        want = sum(q[t, 0, j] * beta[j, 0] * v[j, 0] * torch.prod(dec[j + 1:t + 1, 0]) for j in range(t + 1))
        assert torch.allclose(out[t, 0], want)
    k2 = k.clone()
    k2[3] = k2[1]                                           # token 3 writes under token 1's key
    out2, S2 = O.gated_delta_rule(q, k2, v, torch.ones(T, 1, dtype=torch.float64), torch.ones(T, 1, dtype=torch.float64))
    assert torch.allclose(S2[0, 1], v[3, 0]) and torch.allclose(S2[0, 3], torch.zeros(e, dtype=torch.float64))
    a, Sa = O.gated_delta_rule(q[:4], k[:4], v[:4], beta[:4], dec[:4])
    b, Sb = O.gated_delta_rule(q[4:], k[4:], v[4:], beta[4:], dec[4:], S0=Sa)
    assert torch.allclose(torch.cat([a, b]), out) and torch.allclose(Sb, S)


def test_model_is_causal_and_its_windows_forget():
    cfg = O.small_config([O.attention_layer(window=4, mlp=O.dense(16)), O.latent_layer(window=3)], width=32, vocab=20, side=3)
    sd = O.random_weights(cfg, 1)
    a = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8]
    la, _ = O.forward(cfg, sd, a)
    lb, _ = O.forward(cfg, sd, a[:7] + [0, 0, 0, 0, 0])
    assert torch.allclose(la[:7], lb[:7]) and not torch.allclose(la[7], lb[7])
    lc, _ = O.forward(cfg, sd, [7] + a[1:])                  # two windowed layers see at most 3 + 2 tokens back
    assert torch.allclose(la[6:], lc[6:]) and not torch.allclose(la[5], lc[5])
