"""Daberax on the HIP path against tests/daberax_oracle.py (plain float64 restatement, one function per mechanism).

Small random models of several shapes (all three mixers in different orders, layers without a feed-forward, models without a token
input, sizes that are no multiples of 4 or 8, one head, windows of 1, of a few tokens and longer than any request, no window, no
soft cap, no rotation, partial rotation, rescaled frequencies, one filter tap, twelve query heads on one key head, latents on and
beyond the matrix-core attention's sizes, a recurrence state of 136 rows).  fp32 arithmetic is held to 1e-4 of the logits' scale, the
bf16-MFMA arithmetic to 3e-2.  Covers: every operator alone (attention with scores scaled up until one key decides: at the first
slot, just inside and just outside the window, around key-tile and key-split edges, at the row's own slot, in prompts' runs of rows
and in decode rows, with and without the soft cap; the delta rule row by row and as decode rows on stale, stored and fresh states,
with a write that must survive hundreds of tokens; filter states across differently cut calls); whole prompts with the residual
stream after every layer; token-by-token decoding; portions down to two tokens; several unequal requests in one pass against each
alone; inputs longer than a pass; cache sequences that are released and reused; the first positions of a sequence; long decoding
past every window; the bf16 arithmetic; greedy generation through the generation entry point; the captured decode step; the
trace runner."""
import copy
import ctypes as C
import json
import os
import subprocess

import numpy as np
import pytest
import torch

from tests import daberax_oracle as O

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def config(name):
    A, Lt, Dl, dense = O.attention_layer, O.latent_layer, O.delta_layer, O.dense
    if name == "mixed":     # all mixers, windows of a few tokens, a layer without a feed-forward, rescaled frequencies, soft caps
        return O.small_config([Lt(window=9, mlp=dense(96)), Dl(mlp=dense(48)), Dl(heads=2, kv_heads=1, dim=32, vdim=24, conv=3, mlp=None),
                               A(window=21, softcap=4.0, scaling=(8.0, 1.0, 4.0, 32), mlp=dense(40)), Lt(heads=2, dim=16, rot_dim=4, vdim=8,
                                                                                                         kv_rank=36, softcap=3.0, window=5)])
    if name == "odd":       # no size a multiple of 4 or 8 (every product on the fp32 FMA kernels), partial rotation, other constants
        return O.small_config([A(heads=3, kv_heads=1, dim=10, vdim=18, scale=0.4, rot=(500.0, 6), window=13, mlp=dense(30)),
                               Dl(heads=3, kv_heads=3, dim=10, vdim=6, conv=5, mlp=dense(22)),
                               Lt(heads=3, dim=6, rot_dim=6, vdim=10, kv_rank=17, scale=0.3, base=77.0, window=4, mlp=dense(14))],
                              width=44, vocab=61, side=5, logit_scale=1.7, eps=1e-3)
    if name == "ones":      # values a model may happen to make equal or 1; no token input, no window, no soft cap, no rotation, one tap
        return O.small_config([A(heads=1, kv_heads=1, dim=32, vdim=32, scale=1.0, rot=None, mlp=dense(32)),
                               Dl(heads=1, kv_heads=1, dim=32, vdim=32, conv=1, mlp=dense(32)),
                               Lt(heads=1, dim=32, rot_dim=32, vdim=32, kv_rank=32, scale=1.0, window=1, mlp=dense(32))],
                              width=32, vocab=32, side=0, logit_scale=1.0)
    if name == "wide":      # twelve query heads on one key head, a recurrence state of 136 rows, latents at and beyond the matrix-core sizes
        return O.small_config([A(heads=12, kv_heads=1, dim=8, vdim=8, rot=(10000.0, 8), window=70, mlp=dense(16)),
                               Dl(heads=2, kv_heads=1, dim=136, vdim=40, conv=2, mlp=dense(16)),
                               Lt(heads=5, dim=8, rot_dim=16, vdim=8, kv_rank=200, window=33),
                               Lt(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=260, window=300, mlp=dense(8))], width=32, vocab=40, side=3)
    if name == "tail":      # heads of 72 and 136 values (the matrix-core attention's larger tiles), windows longer than any request
        return O.small_config([Dl(heads=4, kv_heads=4, dim=8, vdim=72), A(heads=2, kv_heads=2, dim=72, vdim=136, scale=0.1, rot=(1e6, 72),
                                                                           softcap=50.0, window=1000, mlp=dense(64)),
                               Dl(heads=4, kv_heads=2, dim=24, vdim=8, conv=4, mlp=dense(64))], width=64, vocab=50, side=8, logit_scale=0.25)
    raise KeyError(name)


MODELS = ("mixed", "odd", "ones", "wide", "tail")


def build(cfg, sd, arith="f32", t_max=512, n_seq=1):
    from ming_univision_amd.configuration import DaberaxConfig
    from ming_univision_amd.daberax import DaberaxDecoder
    return DaberaxDecoder(DaberaxConfig.from_dict(cfg), {k: v.cuda() for k, v in sd.items()}, t_max=t_max, n_seq=n_seq, arith=arith)


def make(name, arith="f32", seed=0, t_max=512, n_seq=1, peaky=1.0):
    cfg = config(name)
    if peaky != 1.0:
        cfg = copy.deepcopy(cfg)
        for ly in cfg["layers"]:
            if ly["type"] != "delta":
                ly["mixer"]["scale"] *= peaky
    sd = O.random_weights(cfg, seed)
    return cfg, sd, build(cfg, sd, arith, t_max, n_seq)


def toks(cfg, n, seed=1):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def err(got, want):
    want = want.double()
    return float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-9))


def ref_logits(cfg, sd, t):
    return O.forward(cfg, sd, t)[0]


def run_spans(dec, ids, spans, trace=False):
    ids = torch.tensor(ids, device="cuda")
    return dec.forward_spans(dec.embed(ids), spans, trace=trace, tokens=ids)


def run_portions(dec, seq, tokens, cuts):
    """Feed `tokens` to cache sequence `seq` in portions of the given sizes; returns the logits of every position."""
    out, at = [], 0
    for n in cuts:
        out.append(dec.logits(run_spans(dec, tokens[at:at + n], [(seq, n, at)])))
        at += n
    assert at == len(tokens)
    return torch.cat(out, 0)


def _api():
    from ming_univision_amd._lib import check, current_stream, lib, ptr
    return check, current_stream, lib(), ptr


def _rows(spans, block_rows=1 << 30):
    from ming_univision_amd.sequences import rows_of_spans
    t = rows_of_spans(spans, block_rows)
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


def dev_freq(rot):
    from ming_univision_amd.daberax import rotary_frequencies
    return rotary_frequencies(rot, "cuda")


# ---- operators alone -------------------------------------------------------------------------------------------------------
def test_rotary_frequencies_in_all_three_bands():
    for rot in ({"base": 10000.0, "dims": 64}, {"base": 300000.0, "dims": 40, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 256}},
                {"base": 100.0, "dims": 6, "scaling": {"factor": 3.0, "low": 0.5, "high": 2.5, "original": 40}}):
        got, ref = dev_freq(rot).cpu().double(), O.rotary_frequencies(rot)
        assert float(((got - ref) / ref).abs().max()) < 1e-7
    sc = {"base": 300000.0, "dims": 40, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 256}}
    plain = O.rotary_frequencies({"base": 300000.0, "dims": 40})
    ratio = O.rotary_frequencies(sc) / plain
    assert float(ratio[0]) == 1.0 and abs(float(ratio[-1]) - 1 / 8.0) < 1e-12 and bool(((ratio > 0.126) & (ratio < 0.999)).any())


def test_result_norm_add_and_gelu_products():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(0)
    for M, n in ((5, 44), (3, 1), (70, 1000), (2, 2100), (3, 8200)):
        x, y, w = torch.randn(M, n + 3, generator=g), 4 * torch.randn(M, n + 1, generator=g), _bf(1 + 0.2 * torch.randn(n, generator=g))
        xd, x16 = x.cuda(), torch.zeros(M, n, dtype=torch.bfloat16, device="cuda")
        check(L.mn_rms_scale_add_rows(ptr(xd), n + 3, ptr(D(y)), n + 1, ptr(D(w)), 1e-3, ptr(x16), n, M, n, stream()))
        ref = x[:, :n].double() + O.rms(y[:, :n].double(), 1e-3) * w.double()
        assert err(xd[:, :n], ref) < 1e-6 and err(x16.float(), ref) < 1e-2 and bool((xd[:, n:].cpu() == x[:, n:]).all())
        a = 2 * torch.randn(M, 2 * n, generator=g)
        out, out16 = torch.zeros(M, n, device="cuda"), torch.zeros(M, n, dtype=torch.bfloat16, device="cuda")
        ad = D(a)
        check(L.mn_gelu_mul_rows(ptr(ad), 2 * n, C.c_void_p(ad.data_ptr() + 4 * n), 2 * n, None, 0, None, ptr(out), n, ptr(out16), n, M, n, stream()))
        ref = O.gelu_tanh(a[:, :n].double()) * a[:, n:].double()
        assert err(out, ref) < 1e-6 and err(out16.float(), ref) < 1e-2
        table, idx = _bf(torch.randn(9, 3 * n + 2, generator=g)), torch.randint(0, 9, (M,), generator=g).to(torch.int32)
        td = D(table)
        check(L.mn_gelu_mul_rows(ptr(ad), 2 * n, None, 0, C.c_void_p(td.data_ptr() + 2 * (n + 1)), 3 * n + 2, ptr(D(idx)), ptr(out), n, None, 0,
                                 M, n, stream()))
        ref = O.gelu_tanh(a[:, :n].double()) * table[idx.long()][:, n + 1:2 * n + 1].double()
        assert err(out, ref) < 1e-6


def test_whole_projection_norms_rotation_and_append():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(1)
    for H, G, d, e, rot in ((4, 2, 16, 16, {"base": 1e4, "dims": 16}), (3, 1, 10, 18, {"base": 500.0, "dims": 6}), (1, 1, 130, 5, None),
                            (5, 5, 64, 72, {"base": 2e5, "dims": 64, "scaling": {"factor": 6.0, "low": 1.0, "high": 3.0, "original": 128}})):
        spans = [(1, 7, 0), (0, 1, 2999), (2, 5, 94)]
        M, t_max, n_seq, eps, scale = 13, 3004, 3, 1e-5, 0.37
        r = _rows(spans)
        nq, nk, nv = H * d, G * d, G * e
        qkv = torch.randn(M, nq + nk + nv + 3, generator=g) * 3
        qw, kw = _bf(1 + 0.2 * torch.randn(nq, generator=g)), _bf(1 + 0.2 * torch.randn(nk, generator=g))
        q = torch.zeros(M, nq, device="cuda")
        ka, va = torch.full((n_seq, t_max, nk), 7.0, device="cuda"), torch.full((n_seq, t_max, nv), 7.0, device="cuda")
        fr = dev_freq(rot) if rot else None
        check(L.mn_proj_norm_rope_append(ptr(D(qkv)), nq + nk + nv + 3, M, H, G, d, e, ptr(D(qw)), ptr(D(kw)), eps, rot["dims"] if rot else 0, 1,
                                         ptr(fr), scale, ptr(r["row_seq"]), ptr(r["row_slot"]), ptr(q), nq, ptr(ka), nk, ptr(va), nv, t_max,
                                         stream()))
        x = qkv.double()
        qr = (O.rms(x[:, :nq], eps) * qw.double()).reshape(M, H, d)
        kr = (O.rms(x[:, nq:nq + nk], eps) * kw.double()).reshape(M, G, d)
        pos = r["row_slot"].cpu().tolist()
        seqs = r["row_seq"].cpu().tolist()
        if rot:
            f = O.rotary_frequencies(rot)
            qr = torch.cat([O.rotate_interleaved(qr[m:m + 1], f, pos[m]) for m in range(M)])
            kr = torch.cat([O.rotate_interleaved(kr[m:m + 1], f, pos[m]) for m in range(M)])
        for m in range(M):
            tol = 2e-5 if pos[m] < 100 else 3e-4                   # an fp32 angle near 3000 radians is rounded to 1.2e-4
            assert err(q[m], qr[m].reshape(-1) * scale) < tol
            assert err(ka[seqs[m], pos[m]], kr[m].reshape(-1)) < tol and err(va[seqs[m], pos[m]], x[m, nq + nk:nq + nk + nv]) < 1e-7
        ka[r["row_seq"].long(), r["row_slot"].long()] = 7.0
        assert bool((ka == 7.0).all())                               # nothing else was written


def attention_case(H, G, d, e, T, window, cap, rows, needle, scale, variant, nsplit=0, one_row=False, seed=0):
    """A sequence of T cached tokens; `rows` = positions of the query rows (consecutive for a run).  needle = (row index, key slot):
    that key is made to dominate that row's scores.  Returns (got, reference) [rows, H, e]."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(seed)
    k, v = torch.randn(T, G, d, generator=g), torch.randn(T, G, e, generator=g)
    q = torch.randn(len(rows), H, d, generator=g)
    if needle is not None:
        ri, slot = needle
        q[ri] = 6.0 * k[slot].repeat_interleave(H // G, 0) / scale / d ** 0.5
    t_max = T + 5
    ka, va = torch.zeros(2, t_max, G * d), torch.zeros(2, t_max, G * e)
    ka[1, :T], va[1, :T] = k.reshape(T, -1), v.reshape(T, -1)
    ka[1, T:], va[1, T:] = 1e4, 1e4                                 # slots past the sequence hold junk that must not be read
    M = len(rows)
    row_seq = torch.ones(M, dtype=torch.int32)
    row_slot = torch.tensor(rows, dtype=torch.int32)
    br = L.mn_window_attn_block_rows()
    blk = torch.tensor([[i, min(br, M - i)] for i in range(0, M, br)], dtype=torch.int32)
    n_blk = M if one_row else blk.shape[0]
    ns = nsplit or L.mn_window_attn_splits(n_blk, H, G, int(one_row), T)
    wsb = L.mn_window_attn_workspace_bytes(n_blk, H, G, e, int(one_row), ns)
    ws = torch.zeros(max(wsb, 16), dtype=torch.uint8, device="cuda")
    out = torch.zeros(M, H * e, device="cuda")
    check(L.mn_window_pool_attn_blocks_cap(ptr(D(q.reshape(M, -1) * scale)), H * d, ptr(D(ka)), 0, ptr(D(va)), 0, None, None, None, cap,
                                           ptr(D(row_seq)), ptr(D(row_slot)), None if one_row else ptr(D(blk)), n_blk, int(one_row), H, G, d, e,
                                           t_max, 1, window, 0, 1.0, ptr(out), H * e, None, 0, ns, ptr(ws), ws.numel(), variant, stream()))
    ref = torch.zeros(M, H, e, dtype=torch.float64)
    for i, p in enumerate(rows):
        lo = max(0, p - window + 1) if window else 0
        for h in range(H):
            s = (k[lo:p + 1, h // (H // G)].double() @ q[i, h].double()) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            ref[i, h] = torch.softmax(s, 0) @ v[lo:p + 1, h // (H // G)].double()
    return out.reshape(M, H, e), ref


@pytest.mark.parametrize("variant", [0, 1])
def test_attention_needles_at_window_tile_and_split_edges(variant):
    """One key decides a row: the first slot, the row's own slot, the oldest slot inside the window (it must be seen) and the one
    before it (it must not), across 16- and 64-key tile edges and forced key splits, in runs of rows of a prompt."""
    for H, G, d, e in ((4, 2, 16, 16), (3, 1, 10, 18), (2, 2, 72, 136)):
        for window, cap in ((0, 0.0), (24, 0.0), (120, 25.0), (17, 5.0), (1, 0.0)):
            T = 300
            rows = [200, 201, 202, 203, 204, 205]                   # two runs: four rows and two rows
            lo = lambda p: max(0, p - window + 1) if window else 0  # noqa: E731
            for ri, slot in ((0, lo(200)), (3, lo(203)), (5, 205), (2, 202 - 15), (4, lo(204) + 63), (1, 0)):
                if slot < 0:
                    continue
                for ns in ((1,) if window == 1 else (1, 3)):
                    got, ref = attention_case(H, G, d, e, T, window, cap, rows, (ri, slot), 0.3, variant, nsplit=ns)
                    assert err(got, ref) < 2e-5, (H, d, window, cap, ri, slot, ns)
            if window > 1:                                           # the slot just outside the window attracts the query but is not seen
                got, ref = attention_case(H, G, d, e, T, window, cap, rows, (0, lo(200) - 1), 0.3, variant)
                assert err(got, ref) < 2e-5


def test_attention_needles_in_decode_rows():
    """The same for rows that are alone in the step (the decode form: key splits and their merge)."""
    for H, G, d, e in ((4, 2, 16, 16), (12, 1, 8, 8), (3, 3, 130, 260)):
        for window, cap in ((0, 0.0), (24, 0.0), (120, 25.0), (17, 0.0)):
            T = 700
            p = 650
            lo = max(0, p - window + 1) if window else 0
            for slot in (lo, lo - 1, p, lo + 63, lo + 64, 0):
                for ns in (0, 1, 5, 64):
                    if slot < 0:
                        continue
                    got, ref = attention_case(H, G, d, e, T, window, cap, [p], (0, slot), 0.3, 1, nsplit=ns, one_row=True)
                    assert err(got, ref) < 2e-5, (H, d, window, slot, ns)


def test_soft_cap_changes_what_a_large_score_weighs():
    """Scores far above the cap all end near the cap: two such keys share the weight, which the uncapped softmax gives to one."""
    got, ref = attention_case(2, 1, 16, 8, 50, 0, 2.0, [40, 41], (0, 7), 3.0, 0)
    got2, ref2 = attention_case(2, 1, 16, 8, 50, 0, 0.0, [40, 41], (0, 7), 3.0, 0)
    assert err(got, ref) < 2e-5 and err(got2, ref2) < 2e-5 and float((ref - ref2).abs().max()) > 0.1


def test_latent_rows_absorbed_attention_against_expanded_heads():
    """The latent layer's operator chain (norm + rotation + append, absorbed queries, attention on [latent ; rotated part] with the
    values a view of the keys, expansion) against per-head keys and values, with a window and a soft cap, stale arena contents."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(3)
    for H, d, r, e, R, window, cap in ((4, 8, 8, 12, 24, 9, 0.0), (3, 6, 6, 10, 17, 4, 2.5), (2, 8, 8, 8, 260, 0, 0.0), (5, 8, 16, 8, 200, 33, 0.0)):
        T, eps, scale, t_max = 60, 1e-5, 0.3, 64
        rot = {"base": 300.0, "dims": r}
        n_in = H * (d + r) + R + r
        x = torch.randn(T, n_in + 1, generator=g) * 2
        cw = _bf(1 + 0.2 * torch.randn(R, generator=g))
        uk, uv = _bf(torch.randn(H * d, R, generator=g) * R ** -0.5), _bf(torch.randn(H * e, R, generator=g) * R ** -0.5)
        ld = L.mn_pn_latent_ld(R, r)
        arena = torch.full((1, t_max, ld), 9.0, device="cuda")
        qf = torch.zeros(T, H * (R + r), device="cuda")
        rows = _rows([(0, T, 0)], L.mn_window_attn_block_rows())
        xd, fr = D(x), dev_freq(rot)
        check(L.mn_latent_rope_append(ptr(xd), n_in + 1, T, H, d, r, R, ptr(D(cw)), eps, r, 1, ptr(fr), scale, ptr(rows["row_seq"]),
                                      ptr(rows["row_slot"]), ptr(qf), H * (R + r), ptr(arena), ld, t_max, stream()))
        ukT = D(uk.reshape(H, d, R).transpose(1, 2).contiguous())
        check(L.mn_gemm_f32_batched(ptr(xd), n_in + 1, d + r, ptr(ukT), d, R * d, None, ptr(qf), H * (R + r), R + r, None, 0, 0, None, 0, 0, T, R, d,
                                    H, scale, stream()))
        lat, out = torch.zeros(T, H * R, device="cuda"), torch.zeros(T, H * e, device="cuda")
        n_blk = rows["blk_tab"].shape[0]
        check(L.mn_window_pool_attn_blocks_cap(ptr(qf), H * (R + r), ptr(arena), ld, ptr(arena), ld, None, None, None, cap, ptr(rows["row_seq"]),
                                               ptr(rows["row_slot"]), ptr(rows["blk_tab"]), n_blk, 0, H, 1, R + r, R, t_max, 1, window, 0, 1.0,
                                               ptr(lat), H * R, None, 0, 1, None, 0, -1, stream()))
        check(L.mn_gemm_f32_batched(ptr(lat), H * R, R, ptr(D(uv)), R, e * R, None, ptr(out), H * e, e, None, 0, 0, None, 0, 0, T, e, R, H, 1.0,
                                    stream()))
        xx = x.double()
        q = xx[:, :H * (d + r)].reshape(T, H, d + r)
        c = O.rms(xx[:, H * (d + r):H * (d + r) + R], eps) * cw.double()
        f = O.rotary_frequencies(rot)
        kr = O.rotate_interleaved(xx[:, H * (d + r) + R:n_in].reshape(T, 1, r), f)
        qq = torch.cat([q[:, :, :d], O.rotate_interleaved(q[:, :, d:].contiguous(), f)], -1)
        kk = torch.cat([(c @ uk.double().T).reshape(T, H, d), kr.expand(T, H, r)], -1)
        ref = O.masked_softmax_attention(qq, kk, (c @ uv.double().T).reshape(T, H, e), scale, window or None, cap or None)
        assert err(out.reshape(T, H, e), ref) < 2e-5, (H, R, window)
        assert err(arena[0, :T, :R], c) < 1e-5 and bool((arena[0, T:] == 9.0).all())


def delta_inputs(g, T, H, G, d, e):
    q, k = torch.randn(T, G, d, generator=g), torch.randn(T, G, d, generator=g)
    q, k = q / q.norm(dim=-1, keepdim=True) * d ** -0.5, k / k.norm(dim=-1, keepdim=True)
    v = torch.randn(T, H, e, generator=g)
    beta, dec = torch.rand(T, H, generator=g), torch.rand(T, H, generator=g) ** 0.1
    return q, k, v, beta, dec


def run_delta(L, check, stream, ptr, q, k, v, beta, dec, state, seq, past, cuts, distinct=False):
    """Rows of one sequence through mn_gated_delta_rows in calls of the given sizes."""
    T, G, d = q.shape
    H, e = v.shape[1], v.shape[2]
    out = torch.zeros(T, H * e, device="cuda")
    at = 0
    for n in cuts:
        sl = slice(at, at + n)
        qkv = torch.cat([q[sl].reshape(n, -1), k[sl].reshape(n, -1), v[sl].reshape(n, -1)], 1)
        bd = torch.cat([beta[sl], dec[sl]], 1)
        r = _rows([(seq, n, past + at)])
        check(L.mn_gated_delta_rows(ptr(D(qkv)), qkv.shape[1], ptr(D(bd)), 2 * H, n, H, G, d, e, ptr(state), ptr(r["row_seq"]), ptr(r["row_slot"]),
                                    ptr(r["row_back"]), 1 if distinct else 0, C.c_void_p(out.data_ptr() + 4 * at * H * e), H * e, stream()))
        at += n
    return out.reshape(T, H, e)


def test_delta_rule_rows_decode_rows_and_states():
    """Row walk and decode rows against the recurrence: a sequence that starts on a stale state (slot 0 reads nothing), continues from
    the stored state across calls cut anywhere, and a second sequence whose state stays untouched; states of 10 .. 500 rows."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(5)
    for H, G, d, e in ((4, 2, 16, 16), (3, 3, 10, 6), (2, 1, 136, 40), (1, 1, 260, 33), (2, 2, 500, 8), (2, 2, 512, 8), (4, 1, 64, 300)):
        T = 45
        q, k, v, beta, dec = delta_inputs(g, T, H, G, d, e)
        rep = H // G
        ref, S = O.gated_delta_rule(q.double().repeat_interleave(rep, 1), k.double().repeat_interleave(rep, 1), v.double(), beta.double(), dec.double())
        for cuts, distinct in (([45], False), ([7, 2, 1, 30, 5], False), ([1] * 45, True), ([20] + [1] * 25, None)):
            state = torch.full((2, H, d, e), 3.0, device="cuda")
            if distinct is None:
                a = run_delta(L, check, stream, ptr, q[:20], k[:20], v[:20], beta[:20], dec[:20], state, 1, 0, [20])
                b = run_delta(L, check, stream, ptr, q[20:], k[20:], v[20:], beta[20:], dec[20:], state, 1, 20, [1] * 25, True)
                got = torch.cat([a, b])
            else:
                got = run_delta(L, check, stream, ptr, q, k, v, beta, dec, state, 1, 0, cuts, distinct)
            assert err(got, ref) < 2e-5, (H, d, e, cuts[:3])
            assert err(state[1], S) < 2e-5 and bool((state[0] == 3.0).all())


def test_delta_rule_keeps_a_write_for_hundreds_of_tokens():
    """Decay 1, full write strength, orthonormal keys: what token 0 wrote under its key is read back unchanged 400 tokens later, in one
    piece, in portions and decoded; with a decay below 1 it has faded by exactly the product of the decays."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(6)
    H, G, d, e, T = 2, 1, 64, 16, 401
    k = torch.zeros(T, G, d)
    k[0, 0, 0] = 1.0
    for t in range(1, T):
        k[t, 0, 1 + (t % (d - 1))] = 1.0                            # never the first direction again
    q = torch.zeros(T, G, d)
    q[:, 0, 0] = 1.0                                                 # every row asks for what token 0 wrote
    v = torch.randn(T, H, e, generator=g)
    beta = torch.ones(T, H)
    for dec_v in (1.0, 0.995):
        dec = torch.full((T, H), dec_v)
        for cuts, distinct in (([T], False), ([100, 2, 299], False), ([1] * T, True)):
            state = torch.full((1, H, d, e), -2.0, device="cuda")
            got = run_delta(L, check, stream, ptr, q, k, v, beta, dec, state, 0, 0, cuts, distinct)
            want = v[0].double() * dec_v ** 400
            assert err(got[400], want) < 1e-5, (dec_v, cuts[:2])


def test_delta_preparation_filters_across_cuts():
    """Filters + silu + unit norms + write strengths + decays of three sequences, fed in calls cut differently, with stale filter
    states in the buffer: every row equals the whole-sequence computation."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(7)
    for H, G, d, e, taps in ((4, 2, 16, 16, 4), (3, 3, 10, 6, 5), (1, 1, 130, 70, 2), (2, 1, 8, 8, 1)):
        nqk, nv = 2 * G * d, H * e
        n = nqk + nv
        ld = n + 2 * H + 3
        lens = {0: 12, 2: 1, 1: 9}
        full = {s: torch.randn(T, ld, generator=g) * 2 for s, T in lens.items()}
        wc = _bf(torch.randn(n, taps, generator=g) * 0.6)
        a_log, dtb = torch.randn(H, generator=g), torch.randn(H, generator=g)
        ref = {}
        for s, x in full.items():
            xx = x.double()
            cv = O.silu(O.causal_conv(xx[:, :n], wc.double()))
            qq, kk = cv[:, :G * d].reshape(-1, G, d), cv[:, G * d:nqk].reshape(-1, G, d)
            qq = qq / torch.sqrt((qq * qq).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
            kk = kk / torch.sqrt((kk * kk).sum(-1, keepdim=True) + 1e-6)
            beta = torch.sigmoid(xx[:, n:n + H])
            dec = torch.exp(-torch.exp(a_log.double()) * O.softplus(xx[:, n + H:n + 2 * H] + dtb.double()))
            ref[s] = (torch.cat([qq.reshape(len(x), -1), kk.reshape(len(x), -1), cv[:, nqk:]], 1), torch.cat([beta, dec], 1))
        for passes in ([[(0, 12, 0), (2, 1, 0), (1, 9, 0)]], [[(0, 5, 0), (1, 2, 0)], [(0, 1, 5), (2, 1, 0), (1, 1, 2)], [(1, 6, 3), (0, 6, 6)]],
                       [[(0, 1, 0), (1, 1, 0)], [(1, 1, 1), (0, 1, 1), (2, 1, 0)], [(0, 10, 2), (1, 7, 2)]]):
            state = torch.full((3, max(taps - 1, 1), n), 50.0, device="cuda")
            for spans in passes:
                M = sum(s[1] for s in spans)
                x = torch.cat([full[s][p:p + c] for s, c, p in spans])
                r = _rows(spans)
                out, bd = torch.zeros(M, n, device="cuda"), torch.zeros(M, 2 * H, device="cuda")
                xd = D(x)
                alone = all(c == 1 for _, c, _ in spans)               # such a call may move the state on by itself
                check(L.mn_delta_prep_rows(ptr(xd), ld, M, H, G, d, e, n, n + H, ptr(D(wc)), taps, ptr(state), int(alone), ptr(D(a_log)),
                                           ptr(D(dtb)), 1e-6, d ** -0.5, ptr(r["row_seq"]), ptr(r["row_slot"]), ptr(r["row_back"]), ptr(out), n,
                                           ptr(bd), 2 * H, stream()))
                if taps > 1 and not alone:
                    check(L.mn_tap_state_update(ptr(xd), ld, taps, ptr(state), ptr(r["row_seq"]), ptr(r["row_back"]), M, n, stream()))
                r0 = 0
                for s, c, p in spans:
                    assert err(out[r0:r0 + c], ref[s][0][p:p + c]) < 2e-5 and err(bd[r0:r0 + c], ref[s][1][p:p + c]) < 2e-5, (taps, spans)
                    r0 += c


def test_head_gates():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(8)
    for M, H, e in ((5, 4, 16), (3, 3, 6), (2, 1, 300), (70, 6, 64)):
        x, gate, w = torch.randn(M, H * e + 2, generator=g) * 3, torch.randn(M, H * e + 1, generator=g), _bf(1 + 0.2 * torch.randn(e, generator=g))
        y, y16 = torch.zeros(M, H * e, device="cuda"), torch.zeros(M, H * e, dtype=torch.bfloat16, device="cuda")
        check(L.mn_head_rms_silu_gate_rows(ptr(D(x)), H * e + 2, ptr(D(w)), 1e-4, ptr(D(gate)), H * e + 1, ptr(y), H * e, ptr(y16), H * e, M, H, e,
                                           stream()))
        ref = (O.rms(x[:, :H * e].double().reshape(M, H, e), 1e-4) * w.double()).reshape(M, -1) * O.silu(gate[:, :H * e].double())
        assert err(y, ref) < 1e-6 and err(y16.float(), ref) < 1e-2
        hg = torch.randn(M, H + 3, generator=g)
        xd = x[:, :H * e].contiguous().cuda()
        check(L.mn_head_sigmoid_gate_rows(ptr(xd), H * e, ptr(D(hg)), H + 3, ptr(y16), H * e, M, H, e, stream()))
        ref = (x[:, :H * e].double().reshape(M, H, e) * torch.sigmoid(hg[:, :H].double())[:, :, None]).reshape(M, -1)
        assert err(xd, ref) < 1e-6 and err(y16.float(), ref) < 1e-2


def test_gelu_product_as_the_streaming_products_epilogue():
    """gelu(x Wg^T) * (x Wu^T) in the epilogue of the weight-streaming product, on its fp32 FMA kernels (1 .. 8 rows) and its matrix-core
    route (more rows, hi/lo operands), against the plain product followed by the activation."""
    from ming_univision_amd import ops
    g = torch.Generator().manual_seed(10)
    for M, N, K in ((1, 40, 64), (3, 320, 200), (8, 96, 2048), (20, 64, 256), (64, 136, 512)):
        x = torch.randn(M, K, generator=g)
        w = _bf(torch.randn(2 * N, K, generator=g) * K ** -0.5)
        got = ops.skinny_gemm(x.cuda(), w.cuda(), epilogue="geglu_tanh")
        y = x.double() @ w.double().T
        ref = O.gelu_tanh(y[:, :N]) * y[:, N:]
        assert got.shape == (M, N) and err(got, ref) < (1e-5 if M <= 8 else 2e-4), (M, N, K)


# ---- whole models ------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", MODELS)
def test_prompt_layers_and_logits(name):
    cfg, sd, dec = make(name)
    t = toks(cfg, 81)
    ref, streams = O.forward(cfg, sd, t)
    hid, tr = run_spans(dec, t, [(0, len(t), 0)], trace=True)
    assert tr.shape[0] == len(cfg["layers"])
    for r in range(tr.shape[0]):
        assert err(tr[r], streams[r]) < 1e-4, r
    assert err(dec.logits(hid), ref) < 1e-4


@pytest.mark.parametrize("name", ["mixed", "odd", "ones"])
def test_first_tokens(name):
    """The first positions: a recurrence and filters from nothing on a reused sequence, a softmax over one key, windows not yet full."""
    cfg, sd, dec = make(name)
    run_portions(dec, 0, toks(cfg, 9, 8), [9])            # leaves keys, latents and states behind
    t = toks(cfg, 6, 5)
    ref = ref_logits(cfg, sd, t)
    assert err(run_portions(dec, 0, t, [1] * 6), ref) < 1e-4
    assert err(run_portions(dec, 0, t, [2, 2, 2]), ref) < 1e-4
    assert err(run_portions(dec, 0, t[:1], [1]), ref[:1]) < 1e-4


@pytest.mark.parametrize("name", MODELS)
def test_portions_and_decoding(name):
    cfg, sd, dec = make(name)
    t = toks(cfg, 150, 2)
    ref = ref_logits(cfg, sd, t)
    tol = 3e-4 if name == "wide" else 1e-4                 # a width of 32 under latents of 200 and 260: small results, divided by their own size
    assert err(run_portions(dec, 0, t, [110] + [1] * 40), ref) < tol                       # prefill against token-by-token decoding
    assert err(run_portions(dec, 0, t, [7, 2, 13, 2, 2, 1, 19, 3, 2, 24, 70, 5]), ref) < tol    # portions cut inside windows and key tiles
    assert err(run_portions(dec, 0, t[:75], [1] * 75), ref[:75]) < tol


def test_single_far_keys_decide_in_prompts_and_decoding():
    """Peaky attention, so that single keys — at the far end of a window, or just inside it — carry the result, in one piece, in
    portions and decoded one by one."""
    for name in ("mixed", "tail"):
        cfg, sd, dec = make(name, peaky=10.0, seed=7)
        t = toks(cfg, 140, 9)
        ref = ref_logits(cfg, sd, t)
        assert err(run_portions(dec, 0, t, [140]), ref) < 2e-4
        assert err(run_portions(dec, 0, t, [80] + [1] * 60), ref) < 2e-4
        assert err(run_portions(dec, 0, t, [9, 3, 4, 5, 11, 2, 30, 66, 10]), ref) < 2e-4


def test_unequal_requests_share_a_pass():
    """Three requests of different lengths in one pass, then a pass that mixes a prompt portion of one with single decode rows of
    the others: every request's logits equal the oracle on that request alone."""
    cfg, sd, dec = make("mixed", n_seq=4)
    reqs = {3: toks(cfg, 120, 1), 0: toks(cfg, 9, 2), 2: toks(cfg, 43, 3)}
    refs = {s: ref_logits(cfg, sd, t) for s, t in reqs.items()}
    first = {3: 70, 0: 8, 2: 42}
    lg = dec.logits(run_spans(dec, [x for s, t in reqs.items() for x in t[:first[s]]], [(s, first[s], 0) for s in reqs]))
    r0 = 0
    for s in reqs:
        assert err(lg[r0:r0 + first[s]], refs[s][:first[s]]) < 1e-4
        r0 += first[s]
    lg = dec.logits(run_spans(dec, [reqs[0][8]] + reqs[3][70:120] + [reqs[2][42]], [(0, 1, 8), (3, 50, 70), (2, 1, 42)]))
    assert err(lg[0:1], refs[0][8:9]) < 1e-4 and err(lg[1:51], refs[3][70:120]) < 1e-4 and err(lg[51:52], refs[2][42:43]) < 1e-4


def test_inputs_longer_than_a_pass(monkeypatch):
    """More rows than one pass through the stack takes: the passes cut a sequence inside a window and a key tile, and a later sequence
    starts inside a pass; the trace is stitched across passes."""
    from ming_univision_amd import seq_lm
    monkeypatch.setattr(seq_lm, "MAX_ROWS", 70)
    cfg, sd, dec = make("mixed", n_seq=2)
    a, b = toks(cfg, 160, 1), toks(cfg, 31, 2)
    (ra, sa), rb = O.forward(cfg, sd, a), ref_logits(cfg, sd, b)
    hid, tr = run_spans(dec, a + b, [(1, 160, 0), (0, 31, 0)], trace=True)
    lg = dec.logits(hid)
    assert err(lg[:160], ra) < 1e-4 and err(lg[160:], rb) < 1e-4 and err(tr[-1][:160], sa[-1]) < 1e-4


def test_released_sequences_are_reused():
    """A cache sequence that held a longer request is given back and reused: its old keys, latents, filter and recurrent states stay in
    memory and must not leak into the next request (nothing is cleared)."""
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
    assert err(run_portions(dec, a, t, [3, 1, 1, 25]), ref_logits(cfg, sd, t)) < 1e-4
    c = slots.alloc()                                     # growing the caches keeps live sequences
    assert c == 2 and dec.n_seq >= 3
    more = toks(cfg, 6, 6)
    assert err(dec.logits(run_spans(dec, more, [(a, 6, 30)])), ref_logits(cfg, sd, t + more)[30:]) < 1e-4
    assert err(dec.logits(run_spans(dec, other[:5], [(b, 5, 0)])), ref_logits(cfg, sd, other[:5])) < 1e-4       # b starts again on its old slots
    dec.release_sequences(2)
    assert err(dec.logits(run_spans(dec, more, [(a, 6, 36)])), ref_logits(cfg, sd, t + more + more)[36:]) < 1e-4  # a lives on after the shrink


def test_long_decoding():
    """300 decoded tokens: every window slides far past the prompt, the recurrent state and the filters are carried by decode rows alone."""
    for name in ("odd", "mixed"):
        cfg, sd, dec = make(name)
        t = toks(cfg, 300, 11)
        assert err(run_portions(dec, 0, t, [5] + [1] * 295), ref_logits(cfg, sd, t)) < 1e-4


def test_bf16_arithmetic():
    """Serving arithmetic: portions above 64 rows take the bf16 MFMA products, portions of 9 .. 64 rows the weight-streaming MFMA route
    on hi/lo rows, rows fed a few at a time fp32 FMA.  The norm on every sublayer's result divides by the result's own size, so a row
    whose result happens to be small amplifies the operands' rounding: rows above 3e-2 of the logits' scale are counted (a few of a
    hundred), none may pass 0.3, and the median row stays below 1e-2."""
    for name in ("mixed", "odd", "wide", "tail"):         # "odd": no K is a multiple of 8
        cfg, sd, dec = make(name, arith="bf16")
        t = toks(cfg, 100)
        ref = ref_logits(cfg, sd, t)
        for cuts in ([100], [70, 21, 9]):
            got = run_portions(dec, 0, t, cuts)
            e = (got.double().cpu() - ref).abs().amax(-1) / ref.abs().max()
            assert int((e > 3e-2).sum()) <= 6 and float(e.max()) < 0.3 and float(e.median()) < 1e-2, (name, cuts, float(e.max()))
        assert err(run_portions(dec, 0, t[:30], [1] * 30), ref[:30]) < 1e-4
        e = (run_portions(dec, 0, t[:64], [12, 20, 32]).double().cpu() - ref[:64]).abs().amax(-1) / ref.abs().max()
        assert float(e.max()) < 2e-2 and float(e.median()) < 2e-3, (name, float(e.max()))


def test_greedy_generation_entry_point():
    """DaberaxForCausalLM.generate: unequal prompts in one lock-step batch; every new token is the oracle's arg-max given the
    tokens before it (or the oracle's two best are within 1e-4), alone or batched, with and without the captured decode step;
    sampled generation returns tokens and gives its cache sequences back."""
    from ming_univision_amd.daberax import DaberaxForCausalLM
    cfg, sd, dec = make("mixed")
    lm = DaberaxForCausalLM(dec)
    prompts = [toks(cfg, 17, 1), toks(cfg, 3, 2), toks(cfg, 40, 3)]
    new = lm.generate(prompts, max_new_tokens=12)
    alone = [lm.generate([p], max_new_tokens=12, use_graph=False)[0] for p in prompts]
    for p, out, solo in zip(prompts, new, alone):
        assert len(out) == 12
        ref = ref_logits(cfg, sd, p + out)
        for i, tok in enumerate(out):
            row = ref[len(p) - 1 + i]
            assert int(row.argmax()) == tok or float(row.max() - row[tok]) < 1e-4
        assert solo == out
    assert not lm.slots.length and lm.slots.next == 3
    out = lm.generate(prompts, max_new_tokens=5, do_sample=True, top_k=8, generator=torch.Generator(device="cuda").manual_seed(0))
    assert all(len(o) == 5 and all(0 <= x < cfg["vocab"] for x in o) for o in out) and not lm.slots.length


def test_decode_graph_replays():
    """The captured decode step against the oracle: every replay is checked (not only the first), with eager work and host
    synchronisations between replays, across a re-capture."""
    cfg, sd, dec = make("mixed", n_seq=3)
    prompts = {0: toks(cfg, 21, 1), 1: toks(cfg, 5, 2), 2: toks(cfg, 30, 3)}
    follow = {s: toks(cfg, 24, 10 + s) for s in prompts}
    refs = {s: ref_logits(cfg, sd, prompts[s] + follow[s]) for s in prompts}
    for s, p in prompts.items():
        run_portions(dec, s, p, [len(p)])
    row_seq = torch.tensor(list(prompts), dtype=torch.int32, device="cuda")
    slot = torch.tensor([len(p) for p in prompts.values()], dtype=torch.int32, device="cuda")
    ln = slot + 1
    g = dec.decode_graph(row_seq, slot, ln)
    g.span = 16                                               # re-capture every 16 tokens
    other = torch.tensor(toks(cfg, 7, 99), device="cuda")
    for i in range(24):
        ids = torch.tensor([follow[s][i] for s in prompts], device="cuda")
        hid = g.run(dec.embed(ids), max(len(p) for p in prompts.values()) + i + 1, tokens=ids)
        lg = dec.logits(hid.clone())
        torch.cuda.synchronize()
        for k, s in enumerate(prompts):
            assert err(lg[k:k + 1], refs[s][len(prompts[s]) + i][None]) < 1e-4, (i, s)
        dec.logits(dec.embed(other))                          # eager work between replays
    assert slot.tolist() == [len(p) + 24 for p in prompts.values()]


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
        ra, rb, rc = (ref_logits(cfg, sd, x) for x in (a, b, c))
        want = {0: ra[[0, 9]], 2: torch.stack([ra[11], rb[5]]), 3: ra[[24]], 4: rc[[0, 10]]}
        assert not (odir / "1.f32").exists()
        for n, ref in want.items():
            got = torch.from_numpy(np.fromfile(odir / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]))
            assert err(got, ref) < tol, (dtype, n)
            os.unlink(odir / f"{n}.f32")
