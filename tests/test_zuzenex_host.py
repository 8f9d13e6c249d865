"""Host-side pieces of the Zuzenex integration that need no GPU: configuration reading and validation, the registry's choice by
config.json, parameter shapes, the order of layer runs, the chunk tables of a pass, and the oracle's own consistency (the sink as an
extra key with a zero value; the recurrence in closed form and in chunked form; the router's pick against its weights)."""
import copy
import json

import numpy as np
import pytest
import torch

from ming_univision_amd.configuration import ZuzenexConfig, config_from_pretrained, zuzenex_param_shapes
from ming_univision_amd.sequences import rows_of_spans
from tests import zuzenex_oracle as O


def small():
    return O.small_config([O.attention_layer(mlp=O.dense(96)), O.lightning_layer(mlp=O.moe(6, 3, 32, identity=2, shared=48)),
                           O.lightning_layer(heads=2, dim=32, vdim=24), O.attention_layer(heads=6, kv_heads=3, dim=8, vdim=24, q_temp=None, mlp=O.moe(4, 2, 24))],
                          loop=(1, 3, 2))


def test_config_and_registry(tmp_path):
    cfg = small()
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    name, c = config_from_pretrained(str(tmp_path))
    assert name == "zuzenex" and isinstance(c, ZuzenexConfig)
    assert (c.width, c.vocab, c.eps) == (64, 80, 1e-5)
    sh = zuzenex_param_shapes(c)
    assert sh == O.param_shapes(cfg)
    assert sh["l0.mix.k"] == (32, 64) and sh["l0.mix.sink"] == (4,) and sh["l0.mix.q.norm"] == (16,) and sh["l0.mlp.up"] == (96, 64)
    assert sh["l1.mlp.router"] == (8, 64) and sh["l1.mlp.correction"] == (8,) and "l1.mlp.e5.up" in sh and "l1.mlp.e6.up" not in sh
    assert sh["l1.mix.g"] == (64, 64) and sh["l2.mix.norm"] == (48,) and sh["l2.mix.o"] == (64, 48) and not any(k.startswith("l2.mlp") for k in sh)
    assert sh["l3.mlp.router"] == (4, 64) and "l3.mlp.shared.up" not in sh and sh["l3.mix.v"] == (72, 64)
    bare = copy.deepcopy(cfg)
    bare.pop("loop")
    assert ZuzenexConfig.from_dict(bare).runs() == [0, 1, 2, 3]


@pytest.mark.parametrize("loop,want", [
    (None, [0, 1, 2, 3]), ((0, 3, 2), [0, 1, 2, 0, 1, 2, 3]), ((1, 2, 3), [0, 1, 1, 1, 2, 3]), ((2, 4, 2), [0, 1, 2, 3, 2, 3]),
    ((0, 4, 1), [0, 1, 2, 3]), ((3, 3, 5), [0, 1, 2, 3])])
def test_order_of_layer_runs(loop, want):
    cfg = small()
    cfg.pop("loop")
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    assert ZuzenexConfig.from_dict(cfg).runs() == want == O.run_order(cfg)


@pytest.mark.parametrize("edit", [
    lambda c: c["layers"][0].update(type="window"), lambda c: c["layers"][0]["mixer"].pop("scale"),
    lambda c: c["layers"][0]["mixer"].update(heads=3), lambda c: c["layers"][1]["mixer"].update(decay=[0.5]),
    lambda c: c["layers"][0]["mlp"].update(kind="gated"), lambda c: c["layers"][1]["mlp"]["router"].update(top=9),
    lambda c: c.update(loop=dict(start=2, stop=1, times=2)), lambda c: c["layers"][0]["mixer"]["q_temp"].update(every=0)])
def test_config_validation(edit):
    cfg = small()
    edit(cfg)
    with pytest.raises(ValueError):
        ZuzenexConfig.from_dict(cfg)


def test_chunk_tables_of_a_pass():
    t = rows_of_spans([(2, 70, 0), (0, 1, 9), (1, 33, 64)], 4, 32)
    assert t["chunk_tab"].tolist() == [[0, 32], [32, 32], [64, 6], [70, 1], [71, 32], [103, 1]]
    assert t["blk_tab"][:2].tolist() == [[0, 4], [4, 4]] and t["blk_tab"][17].tolist() == [68, 2] and t["max_len"] == 97
    assert "chunk_tab" not in rows_of_spans([(0, 3, 0)], 4)
    assert np.array_equal(t["row_back"][68:73], [68, 69, 0, 0, 1])


def test_sink_is_a_key_with_no_value():
    g = torch.Generator().manual_seed(0)
    T, H, G, d, e = 9, 4, 2, 6, 5
    q, k, v = (torch.randn(T, n, c, generator=g, dtype=torch.float64) for n, c in ((H, d), (G, d), (G, e)))
    sink = torch.tensor([0.3, -2.0, 5.0, 0.0], dtype=torch.float64)
    got = O.sink_softmax_attention(q, k, v, sink, 0.7)
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    for h in range(H):
        s = ((q[:, h] @ k[:, h // 2].T) * 0.7).masked_fill(~mask, float("-inf"))
        p = torch.softmax(torch.cat([s, sink[h].expand(T, 1)], 1), -1)            # the sink as one more column ...
        assert torch.allclose(p[:, :T] @ v[:, h // 2], got[:, h], atol=1e-12)      # ... whose value is zero
    none = O.sink_softmax_attention(q, k, v, torch.full((H,), -float("inf"), dtype=torch.float64), 0.7)
    assert torch.allclose(none[0], v[0].repeat_interleave(2, 0), atol=1e-12)       # position 0 without a sink returns its own value


def test_query_temperature_steps():
    t = O.query_temperature(10, {"coef": 0.5, "every": 4})
    assert torch.allclose(t[:3], torch.ones(3, dtype=torch.float64)) and abs(float(t[3]) - (1 + 0.5 * np.log(2.0))) < 1e-12
    assert float(t[6]) == float(t[3]) and abs(float(t[7]) - (1 + 0.5 * np.log(3.0))) < 1e-12
    assert torch.equal(O.query_temperature(5, {"coef": 0.5, "every": 4}, pos0=5), t[5:])
    assert torch.equal(O.query_temperature(4, None), torch.ones(4, dtype=torch.float64))


def test_recurrence_in_closed_and_chunked_form():
    g = torch.Generator().manual_seed(1)
    T, H, d, e = 11, 3, 4, 5
    q, k, v = (torch.randn(T, H, c, generator=g, dtype=torch.float64) for c in (d, d, e))
    lam = torch.tensor([0.5, 1.0, 0.97], dtype=torch.float64)
    out, S = O.lightning_recurrence(q, k, v, lam)
    for h in range(H):                                      # o_t = sum_(j <= t) lam^(t - j) (q_t . k_j) v_j
        for t in (0, 4, T - 1):
            ref = sum(lam[h] ** (t - j) * (q[t, h] @ k[j, h]) * v[j, h] for j in range(t + 1))
            assert torch.allclose(out[t, h], ref, atol=1e-12)
    a, Sa = O.lightning_recurrence(q[:6], k[:6], v[:6], lam)             # cut in two: the state carries everything
    b, Sb = O.lightning_recurrence(q[6:], k[6:], v[6:], lam, Sa)
    assert torch.allclose(torch.cat([a, b]), out, atol=1e-12) and torch.allclose(Sb, S, atol=1e-12)


def test_router_picks_by_corrected_scores_and_weighs_by_scores():
    h = torch.eye(4, dtype=torch.float64)
    router = torch.tensor([[2.0, 0, 0, 0], [1.0, 0, 0, 0], [0.0, 0, 0, 0]], dtype=torch.float64).T.contiguous().T   # outputs 0..2 read h[0]
    corr = torch.tensor([0.0, 0.0, 1.0], dtype=torch.float64)
    idx, w, s = O.route(h[:1], router, corr, 2)
    assert idx.tolist() == [[2, 0]]                                        # the correction lifts output 2 over output 1 ...
    assert torch.allclose(w, torch.stack([s[0, 2], s[0, 0]])[None] / (s[0, 2] + s[0, 0]))      # ... but the weights are the plain scores
    cfg = O.small_config([O.lightning_layer(mlp=O.moe(2, 3, 8, identity=1))], width=16, vocab=8)
    sd = {k: v.double() for k, v in O.random_weights(cfg).items()}
    x = torch.randn(5, 16, dtype=torch.float64)
    y = O.feed_forward(x, sd, "l0.mlp.", cfg["layers"][0]["mlp"])           # every output chosen: sum_i s_i expert_i + s_pass x
    s = torch.softmax(x @ sd["l0.mlp.router"].T, -1)
    ref = s[:, 2:3] * x + sum(s[:, i:i + 1] * O.expert(x, sd[f"l0.mlp.e{i}.up"], sd[f"l0.mlp.e{i}.down"]) for i in range(2))
    assert torch.allclose(y, ref, atol=1e-12)
