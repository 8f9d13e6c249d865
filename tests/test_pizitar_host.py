"""Host-side pieces of the Pizitar integration that need no GPU: configuration reading and validation, the registry's choice by
config.json, parameter shapes, cache-sequence numbering, the per-row tables of a pass, and the oracle's own consistency."""
import json

import numpy as np
import pytest
import torch

from ming_univision_amd.configuration import (MODEL_REGISTRY, MingUniVisionConfig, PizitarConfig, config_from_pretrained,
                                              pizitar_param_shapes)
from ming_univision_amd.sequences import SequenceSlots, rows_of_spans
from tests import pizitar_oracle as O

LAYERS = [dict(type="latent_attention", heads=3, dim=24, vdim=16, kv_rank=40, q_rank=20, ff=72),
          dict(type="latent_attention_2", heads=2, dim=16, vdim=24, kv_rank=72, ff=None),
          dict(type="latent_attention", heads=2, dim=8, vdim=8, kv_rank=40, q_rank=12, kv_from=0, ff=30)]


def test_config_and_registry(tmp_path):
    cfg = O.random_config(LAYERS, width=48, vocab=67, taps=3)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    name, c = config_from_pretrained(str(tmp_path))
    assert name == "pizitar" and isinstance(c, PizitarConfig)
    assert (c.width, c.vocab, c.taps, c.eps, c.logit_softcap) == (48, 67, 3, 1e-5, 20.0)
    assert pizitar_param_shapes(c) == O.tensor_shapes(cfg)
    sh = pizitar_param_shapes(c)
    assert "l2.mix.dkv" not in sh and "l1.mlp.up" not in sh and "l1.rg2" not in sh and sh["l0.mix.uk"] == (72, 40)
    (tmp_path / "config.json").write_text(MingUniVisionConfig.ming_univision_16b_a3b().to_json_string())
    assert config_from_pretrained(str(tmp_path))[0] == "ming_univision"
    (tmp_path / "config.json").write_text(json.dumps({"architecture": "Other"}))
    with pytest.raises(ValueError):
        config_from_pretrained(str(tmp_path))
    assert [n for n, _, _ in MODEL_REGISTRY] == ["pizitar", "sakinex", "zuzenex", "daberax", "ming_univision"]


@pytest.mark.parametrize("edit", [
    lambda L: L[2]["mixer"].update(kv_from=2), lambda L: L[2]["mixer"].update(kv_from=1, kv_rank=40),
    lambda L: L[0].update(type="window"), lambda L: L[0]["mixer"].pop("q_rank"), lambda L: L[0]["mlp"].update(kind="moe"),
    lambda L: L[1]["mixer"].update(kv_from=0)])
def test_config_validation(edit):
    cfg = O.random_config(LAYERS)
    edit(cfg["layers"])
    with pytest.raises(ValueError):
        PizitarConfig.from_dict(cfg)


class _Arena:
    n_seq = 1

    def ensure_sequences(self, n):
        self.n_seq = max(self.n_seq, n)


def test_sequence_slots():
    dec = _Arena()
    s = SequenceSlots(dec, first=1)
    a, b, c = s.alloc(), s.alloc(), s.alloc()
    assert (a, b, c) == (1, 2, 3) and dec.n_seq == 4
    s.length[b] = 7
    s.release(b)
    s.release(a)
    assert s.alloc() == 1 and s.alloc() == 2 and s.length[2] == 0 and s.alloc() == 4
    with pytest.raises(KeyError):
        s.release(9)
    assert s.live_tokens() == 0


def test_rows_of_spans():
    t = rows_of_spans([(5, 6, 10), (2, 1, 0), (7, 9, 3)], 4)
    assert t["row_seq"].tolist() == [5] * 6 + [2] + [7] * 9
    assert t["row_slot"].tolist() == list(range(10, 16)) + [0] + list(range(3, 12))
    assert t["row_back"].tolist() == list(range(6)) + [0] + list(range(9))
    assert (t["row_len"] == t["row_slot"] + 1).all() and t["max_len"] == 16
    assert t["blk_tab"].tolist() == [[0, 4], [4, 2], [6, 1], [7, 4], [11, 4], [15, 1]]
    assert all(v.dtype == np.int32 for k, v in t.items() if k != "max_len")


def test_oracle_is_causal_and_consistent():
    """The oracle evaluates whole sequences; a prefix evaluated alone must give the same logits (nothing looks ahead), and the
    expanded-head attention equals the absorbed form the kernels use."""
    cfg = O.random_config(LAYERS, width=48, vocab=67, taps=3)
    sd = O.random_weights(cfg, 0)
    t = torch.randint(0, 67, (20,), generator=torch.Generator().manual_seed(0)).tolist()
    full, part = O.logits_of(cfg, sd, t), O.logits_of(cfg, sd, t[:11])
    assert float((full[:11] - part).abs().max()) < 1e-9
    g = torch.Generator().manual_seed(1)
    H, d, v, r, T = 2, 6, 5, 7, 9
    q, c = torch.randn(T, H * d, generator=g, dtype=torch.float64), torch.randn(T, r, generator=g, dtype=torch.float64)
    uk, uv = torch.randn(H * d, r, generator=g, dtype=torch.float64), torch.randn(H * v, r, generator=g, dtype=torch.float64)
    ref = O.latent_attention_core(q, c, uk, uv, H, d, v, 0.3)
    for h in range(H):
        qa = 0.3 * q[:, h * d:(h + 1) * d] @ uk[h * d:(h + 1) * d]
        s = (qa @ c.T).masked_fill(torch.ones(T, T).triu(1).bool(), float("-inf"))
        out = (torch.softmax(s, -1) @ c) @ uv[h * v:(h + 1) * v].T
        assert float((out - ref[:, h * v:(h + 1) * v]).abs().max()) < 1e-12
