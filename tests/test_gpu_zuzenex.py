"""Zuzenex on the HIP path against tests/zuzenex_oracle.py (plain float64 restatement, one function per mechanism).

Small random models of several shapes (both mixers with every kind of feed-forward, layers without one, sizes that are no multiples
of 8, one head, as many key/value heads as query heads, twelve query heads on one key/value head, heads of other key and value
sizes, recurrence states of 136 and 260 rows, no query temperature and one that steps at every position, no pass-through outputs,
no shared expert, every router output chosen, more experts than the sorted route takes, repeated ranges at the start / middle / end /
not at all).  fp32 arithmetic is held to 1e-4 of the logits' scale, the bf16-MFMA arithmetic to 3e-2.  Covers: every operator alone
(attention with scores scaled up until one key decides: at the first slot, around key-tile and key-split edges, at the row's own
slot, and one slot past it; sinks that take nearly all or nearly none of the softmax; the recurrence row by row, as decode rows and
as the chunked scan with sequences starting, continuing and ending inside chunks; the router with corrections that change the
pick, ties and pass-through outputs); whole prompts with the residual stream after every layer run; token-by-token decoding;
portions down to two tokens; several unequal requests in one pass against each alone; inputs longer than a pass; cache sequences
that are released and reused; the first positions of a sequence; long decoding; the bf16 arithmetic; greedy generation through the
generation entry point; the captured decode step; the trace runner."""
import copy
import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

from tests import zuzenex_oracle as O

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def config(name):
    A, Lt, dense, moe = O.attention_layer, O.lightning_layer, O.dense, O.moe
    if name == "mixed":     # both mixers with every feed-forward kind, a layer without one, a repeated middle range
        return O.small_config([A(mlp=dense(96)), Lt(mlp=moe(6, 3, 32, identity=2, shared=48)), Lt(heads=2, dim=32, vdim=24, mlp=None),
                               A(heads=6, kv_heads=3, dim=8, vdim=24, q_temp=None, mlp=moe(4, 2, 24)), Lt(mlp=dense(40))], loop=(1, 3, 2))
    if name == "odd":       # no size a multiple of 8 (every product on the fp32 FMA kernels), every router output chosen
        return O.small_config([Lt(heads=3, dim=10, vdim=6, decay=[0.3, 0.95, 1.0], mlp=moe(3, 4, 50, identity=1, shared=10)),
                               A(heads=3, kv_heads=1, dim=10, vdim=18, scale=0.4, q_temp=(0.25, 3), mlp=dense(30))], width=44, vocab=61)
    if name == "ones":      # values a model may happen to make equal or 1
        return O.small_config([A(heads=1, kv_heads=1, dim=32, vdim=32, scale=1.0, q_temp=(1.0, 1), mlp=moe(1, 1, 32, identity=1, shared=32)),
                               Lt(heads=1, dim=32, vdim=32, decay=[1.0], mlp=moe(2, 1, 32))], width=32, vocab=32, loop=(0, 2, 1))
    if name == "wide":      # twelve query heads on one key/value head, a recurrence state of 136 rows, more experts than the sorted route
        return O.small_config([A(heads=12, kv_heads=1, dim=8, vdim=8, mlp=moe(130, 4, 8, identity=3, shared=8)),
                               Lt(heads=2, dim=136, vdim=40, mlp=dense(16))], width=32, vocab=40, loop=(0, 1, 3))
    if name == "tail":      # the repeated range at the end, heads of 64 and 128 values (the matrix-core attention's larger tiles)
        return O.small_config([Lt(heads=2, dim=24, vdim=8), A(heads=2, kv_heads=2, dim=72, vdim=136, scale=0.1, q_temp=(0.1, 16), mlp=dense(64)),
                               Lt(heads=4, dim=8, vdim=16, mlp=moe(5, 2, 64, identity=1))], width=64, vocab=50, loop=(1, 3, 2))
    raise KeyError(name)


MODELS = ("mixed", "odd", "ones", "wide", "tail")


def build(cfg, sd, arith="f32", t_max=512, n_seq=1):
    from ming_univision_amd.configuration import ZuzenexConfig
    from ming_univision_amd.zuzenex import ZuzenexDecoder
    return ZuzenexDecoder(ZuzenexConfig.from_dict(cfg), {k: v.cuda() for k, v in sd.items()}, t_max=t_max, n_seq=n_seq, arith=arith)


def make(name, arith="f32", seed=0, t_max=512, n_seq=1, peaky=1.0):
    cfg = config(name)
    if peaky != 1.0:
        cfg = copy.deepcopy(cfg)
        for ly in cfg["layers"]:
            if ly["type"] == "attention":
                ly["mixer"]["scale"] *= peaky
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


def _rows(spans, block_rows=1 << 30, chunk_rows=0):
    from ming_univision_amd.sequences import rows_of_spans
    t = rows_of_spans(spans, block_rows, chunk_rows)
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
def test_head_norm_temperature_append():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(0)
    for H, G, d, e, coef, every in ((4, 2, 16, 16, 0.5, 8), (3, 1, 10, 18, 0.25, 3), (1, 1, 130, 5, 1.0, 1), (2, 2, 512, 64, 0.0, 0), (5, 5, 64, 72, 2.0, 100)):
        spans = [(1, 7, 0), (0, 1, 299), (2, 5, 94)]
        M, t_max, n_seq, eps, scale = 13, 304, 3, 1e-5, 0.37
        r = _rows(spans)
        C_ = (H + G) * d + G * e
        qkv = torch.randn(M, C_ + 3, generator=g) * 3
        qw, kw = _bf(1 + 0.2 * torch.randn(d, generator=g)), _bf(1 + 0.2 * torch.randn(d, generator=g))
        q = torch.zeros(M, H * d, device="cuda")
        ka, va = torch.full((n_seq, t_max, G * d), 7.0, device="cuda"), torch.full((n_seq, t_max, G * e), 7.0, device="cuda")
        check(L.mn_head_norm_temp_append(ptr(D(qkv)), C_ + 3, M, H, G, d, e, ptr(D(qw)), ptr(D(kw)), eps, scale, coef, every, ptr(r["row_seq"]),
                                         ptr(r["row_slot"]), ptr(q), H * d, ptr(ka), ptr(va), t_max, stream()))
        x = qkv.double()
        pos = r["row_slot"].cpu()
        temp = torch.stack([O.query_temperature(1, {"coef": coef, "every": every} if every else None, int(p))[0] for p in pos])
        qr = O.rms_norm(x[:, :H * d].reshape(M, H, d), O.f64(qw), eps) * temp[:, None, None] * scale
        kr = O.rms_norm(x[:, H * d:(H + G) * d].reshape(M, G, d), O.f64(kw), eps)
        assert err(q, qr.reshape(M, -1)) < 1e-5
        seq = r["row_seq"].cpu().long()
        assert err(ka[seq, pos.long()], kr.reshape(M, -1)) < 1e-5
        assert torch.equal(va[seq, pos.long()].cpu(), qkv[:, (H + G) * d:C_])
        untouched = torch.ones(n_seq, t_max, dtype=torch.bool)
        untouched[seq, pos.long()] = False
        assert bool((ka.cpu()[untouched] == 7.0).all()) and bool((va.cpu()[untouched] == 7.0).all())


def _attention(L, check, ptr, stream, q, ka, va, sink, spans, H, G, d, e, one_row, nsplit, variant):
    """The block attention over rows described by spans -> [M, H * e]."""
    M = q.shape[0]
    r = _rows(spans, L.mn_window_attn_block_rows())
    n_blk = M if one_row else r["blk_tab"].shape[0]
    ws = torch.empty(max(16, L.mn_window_attn_workspace_bytes(n_blk, H, G, e, int(one_row), nsplit)), dtype=torch.uint8, device="cuda")
    out = torch.zeros(M, H * e, device="cuda")
    check(L.mn_window_pool_attn_blocks_sink(ptr(q), H * d, ptr(ka), ptr(va), None, None, ptr(sink) if sink is not None else None, ptr(r["row_seq"]),
                                            ptr(r["row_slot"]), None if one_row else ptr(r["blk_tab"]), n_blk, int(one_row), H, G, d, e, ka.shape[1],
                                            1, 0, 0, 1.0, ptr(out), H * e, None, 0, nsplit, ptr(ws), ws.numel(), variant, stream()))
    return out


@pytest.mark.parametrize("H,G,d,e", [(4, 2, 16, 16), (3, 1, 10, 18), (12, 1, 8, 8), (2, 2, 72, 136), (1, 1, 260, 20)])
def test_sink_attention_needles_at_tile_and_split_edges(H, G, d, e):
    """One key far outweighs the others for one query: the output must be that key's value when it is at or before the query's own
    slot, and must not change when it lies one slot past it.  Needles sit at slot 0, around the 16- / 64-key tile edges, around forced
    key-split edges and at the last visible slot; a sink in between is part of the expected softmax."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(1)
    T, rep = 200, H // G
    ka, va = torch.randn(1, T, G * d, generator=g), torch.randn(1, T, G * e, generator=g)
    sink = torch.randn(H, generator=g)
    for needle in (0, 15, 16, 17, 63, 64, 65, 127, 128, 198, 199):
        k2 = ka.clone()
        qv = torch.randn(H, d, generator=g)
        for h in range(H):                                  # every head's query points at the needle key of its group
            k2[0, needle, (h // rep) * d:(h // rep + 1) * d] = 0
        for grp in range(G):
            k2[0, needle, grp * d:(grp + 1) * d] = 6.0 * qv[grp * rep] / qv[grp * rep].norm()
        for h in range(H):
            qv[h] = qv[(h // rep) * rep] * (1.0 + 0.1 * (h % rep))
        for pos_q in sorted({needle - 1, needle, needle + 1, T - 1} - {-1, T}):
            n_rows = min(4, pos_q + 1)                      # a run of rows ending at pos_q (matrix-core kernel), and pos_q alone (decode kernel)
            q = qv.reshape(1, -1).repeat(n_rows, 1) * 3.0
            kk = O.f64(k2[0]).reshape(T, G, d)
            vv = O.f64(va[0]).reshape(T, G, e)
            same_q = O.f64(q[:1]).reshape(1, H, d).expand(pos_q + 1, H, d)      # causal: row p of the result is position p's view
            ref = O.sink_softmax_attention(same_q, kk[:pos_q + 1], vv[:pos_q + 1], O.f64(sink), 1.0)[pos_q - n_rows + 1:].reshape(n_rows, -1)
            for one_row, variant, splits in ((False, 0 if max(d, e) <= 256 else 1, (1, 3)), (False, 1, (1,)), (True, 1, (1, 3, 64))):
                for ns in splits:
                    spans = [(0, 1, pos_q)] if one_row else [(0, n_rows, pos_q - n_rows + 1)]
                    qq = q[-1:] if one_row else q
                    out = _attention(L, check, ptr, stream, D(qq), D(k2), D(va), D(sink), spans, H, G, d, e, one_row, ns, variant)
                    assert err(out, ref[-1:] if one_row else ref) < 2e-5, (needle, pos_q, one_row, variant, ns)


def test_sink_takes_all_or_nothing():
    """A sink far above every score leaves almost nothing of the values; one far below changes nothing; no sink pointer = no sink."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(2)
    H, G, d, e, T = 4, 2, 16, 24, 70
    ka, va, q = torch.randn(1, T, G * d, generator=g), torch.randn(1, T, G * e, generator=g), torch.randn(6, H * d, generator=g)
    spans = [(0, 6, T - 6)]
    kk, vv = O.f64(ka[0]).reshape(T, G, d), O.f64(va[0]).reshape(T, G, e)

    def ref(sink):
        qs = torch.zeros(T, H, d, dtype=torch.float64)
        qs[T - 6:] = O.f64(q).reshape(6, H, d)
        return O.sink_softmax_attention(qs, kk, vv, sink, 1.0)[T - 6:].reshape(6, -1)
    for sink in (torch.tensor([40.0, -40.0, 0.0, 3.0]), torch.tensor([-1e4, 90.0, -3.0, 0.5])):
        for one_row in (False, True):
            sp = [(0, 1, T - 1)] if one_row else spans
            out = _attention(L, check, ptr, stream, D(q[-1:] if one_row else q), D(ka), D(va), D(sink), sp, H, G, d, e, one_row, 2, -1)
            r = ref(O.f64(sink))
            assert float((out.double().cpu() - (r[-1:] if one_row else r)).abs().max()) < 2e-5
    out = _attention(L, check, ptr, stream, D(q), D(ka), D(va), None, spans, H, G, d, e, False, 1, -1)
    assert float((out.double().cpu() - ref(torch.full((H,), -math.inf, dtype=torch.float64))).abs().max()) < 2e-5


def _light_ref(qkv, H, d, e, decay, spans, S_init):
    """Oracle outputs and final states of the recurrence for rows given as spans; S_init {seq: [H, d, e]} for spans that continue."""
    x = O.silu(O.f64(qkv))
    outs, fin, r0 = [], {}, 0
    for seq, n, past in spans:
        rows = x[r0:r0 + n]
        q, k, v = rows[:, :H * d].reshape(n, H, d), rows[:, H * d:2 * H * d].reshape(n, H, d), rows[:, 2 * H * d:2 * H * d + H * e].reshape(n, H, e)
        o, S = O.lightning_recurrence(q, k, v, O.f64(decay), None if past == 0 else S_init[seq])
        outs.append(o.reshape(n, -1))
        fin[seq] = S
        r0 += n
    return torch.cat(outs), fin


@pytest.mark.parametrize("H,d,e", [(4, 16, 16), (3, 10, 6), (2, 136, 40), (1, 260, 12), (2, 64, 300), (2, 128, 128)])
def test_lightning_recurrence_rows_steps_and_scan(H, d, e):
    """The recurrence three ways against the oracle: row by row, as decode rows (every row alone in its sequence), and as the chunked
    scan — with sequences that start at position 0 (stale state in the arena must not be read), that continue from a stored state, and
    that start, continue and end inside chunks; the state each leaves is checked too."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(3)
    decay = torch.tensor([0.05, 1.0, 0.999, 0.6][:H] + [0.9] * max(0, H - 4))
    n_seq, C_ = 4, 2 * H * d + H * e
    stale = torch.randn(n_seq, H, d, e, generator=g)
    spans = [(2, 70, 0), (0, 33, 5), (3, 1, 0), (1, 45, 64)]
    M = sum(n for _, n, _ in spans)
    qkv = torch.randn(M, C_ + 1, generator=g)
    ref, fin = _light_ref(qkv[:, :C_], H, d, e, decay, spans, {s: O.f64(stale[s]) for s in range(n_seq)})
    chunk = L.mn_lightning_chunk_rows()
    r = _rows(spans, chunk_rows=chunk)
    lds_ok = L.mn_lightning_scan_lds_bytes(d, e) <= 64 * 1024
    for mode in ("rows", "scan", "scan_valu"):               # "scan": the matrix-core output pass where its tiles fit
        if mode != "rows" and not lds_ok:
            continue
        state, out = stale.clone().cuda(), torch.zeros(M, H * e, device="cuda")
        if mode == "rows":
            check(L.mn_lightning_rows(ptr(D(qkv)), C_ + 1, M, H, d, e, ptr(D(decay)), ptr(state), ptr(r["row_seq"]), ptr(r["row_slot"]),
                                      ptr(r["row_back"]), 0, ptr(out), H * e, stream()))
        else:
            n_ch = r["chunk_tab"].shape[0]
            ws = torch.empty(L.mn_lightning_scan_workspace_bytes(n_ch, H, d, e), dtype=torch.uint8, device="cuda")
            if mode == "scan":
                check(L.mn_lightning_rows_scan(ptr(D(qkv)), C_ + 1, M, H, d, e, ptr(D(decay)), ptr(state), ptr(r["row_seq"]), ptr(r["row_slot"]),
                                               ptr(r["row_back"]), ptr(r["chunk_tab"]), n_ch, ptr(out), H * e, ptr(ws), ws.numel(), stream()))
            else:
                check(L.mn_lightning_rows_scan_ex(ptr(D(qkv)), C_ + 1, M, H, d, e, ptr(D(decay)), ptr(state), ptr(r["row_seq"]), ptr(r["row_slot"]),
                                                  ptr(r["row_back"]), ptr(r["chunk_tab"]), n_ch, ptr(out), H * e, ptr(ws), ws.numel(), 1, stream()))
        assert err(out, ref) < 2e-5, mode
        for s, S in fin.items():
            assert err(state[s], S) < 2e-5, (mode, s)
    # decode rows: one row per sequence, one of them at position 0
    rows1 = [(0, 1, 9), (1, 1, 0), (3, 1, 2)]
    q1 = torch.randn(3, C_, generator=g)
    ref1, fin1 = _light_ref(q1, H, d, e, decay, rows1, {s: O.f64(stale[s]) for s in range(n_seq)})
    r1 = _rows(rows1)
    state, out = stale.clone().cuda(), torch.zeros(3, H * e, device="cuda")
    check(L.mn_lightning_rows(ptr(D(q1)), C_, 3, H, d, e, ptr(D(decay)), ptr(state), ptr(r1["row_seq"]), ptr(r1["row_slot"]), None, 1, ptr(out),
                              H * e, stream()))
    assert err(out, ref1) < 2e-5
    for s, S in fin1.items():
        assert err(state[s], S) < 2e-5
    assert torch.equal(state[2].cpu(), stale[2])                 # a sequence without a row keeps its state


def test_gate_norm_and_activation_rows():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(4)
    for M, n in ((1, 44), (5, 256), (3, 1000), (2, 4100)):
        x, gt, w = torch.randn(M, n + 2, generator=g) * 3, torch.randn(M, n + 1, generator=g) * 2, _bf(1 + 0.2 * torch.randn(n, generator=g))
        y, y16 = torch.zeros(M, n, device="cuda"), torch.zeros(M, n, dtype=torch.bfloat16, device="cuda")
        check(L.mn_rms_sigmoid_gate_rows(ptr(D(x)), n + 2, ptr(D(w)), 1e-5, ptr(D(gt)), n + 1, ptr(y), n, ptr(y16), n, M, n, stream()))
        ref = O.rms_norm(O.f64(x[:, :n]), O.f64(w), 1e-5) * torch.sigmoid(O.f64(gt[:, :n]))
        assert err(y, ref) < 1e-5 and err(y16.float(), ref) < 5e-3
        check(L.mn_relu2_rows(ptr(D(x)), n + 2, ptr(y), n, ptr(y16), n, M, n, stream()))
        assert err(y, O.relu2(O.f64(x[:, :n]))) < 1e-6 and err(y16.float(), O.relu2(O.f64(x[:, :n]))) < 5e-3


def test_router_scores_correction_picks_and_pass_through():
    """Softmax over every output, the pick by score + correction (a correction that lifts a low score into the pick and one that
    pushes the highest out), weights from the scores alone over their sum, ties to the lower index, outputs past the experts written
    as one pass-through index; up to 300 outputs and 70 picks; the activation riding the same launch."""
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(5)
    for M, n, n_real, top in ((7, 18, 16, 3), (3, 4, 3, 4), (5, 2, 1, 1), (9, 133, 130, 4), (4, 300, 290, 70), (6, 8, 8, 2)):
        z = torch.randn(M, n + 3, generator=g) * 2
        corr = 0.05 * torch.randn(n, generator=g)
        corr[0], corr[n - 1] = 2.0, -2.0                       # output 0 is always picked, the last never unless everything is
        rx = torch.randn(M, 37, generator=g)
        idx, w = torch.zeros(M, top, dtype=torch.int32, device="cuda"), torch.zeros(M, top, device="cuda")
        ry = torch.zeros(M, 30, device="cuda")
        check(L.mn_router_softmax_topk_rows(ptr(D(z)), n + 3, M, n, n_real, top, ptr(D(corr)), ptr(idx), ptr(w), ptr(D(rx)), 37, ptr(ry), 30, 30, stream()))
        s = torch.softmax(O.f64(z[:, :n]), -1)
        ri = torch.topk(s + O.f64(corr), top, dim=-1).indices
        rw = torch.gather(s, 1, ri)
        rw = rw / (rw.sum(-1, keepdim=True) + 1e-20)
        assert torch.equal(idx.cpu().long(), ri.clamp_max(n_real)), (n, top)
        assert err(w, rw) < 1e-5
        assert bool((idx.cpu()[:, 0] == 0).all())
        assert err(ry, O.relu2(O.f64(rx[:, :30]))) < 1e-6
    z = torch.zeros(2, 6)                                       # equal scores everywhere: the lowest indices win
    idx, w = torch.zeros(2, 3, dtype=torch.int32, device="cuda"), torch.zeros(2, 3, device="cuda")
    check(L.mn_router_softmax_topk_rows(ptr(D(z)), 6, 2, 6, 6, 3, None, ptr(idx), ptr(w), None, 0, None, 0, 0, stream()))
    assert idx.cpu().tolist() == [[0, 1, 2]] * 2 and err(w, torch.full((2, 3), 1 / 3)) < 1e-6


def test_indexed_products_skip_pass_through_and_combine_adds_the_input():
    check, stream, L, ptr = _api()
    g = torch.Generator().manual_seed(6)
    M, top, n, K_, E = 5, 3, 24, 16, 4
    a, w = torch.randn(M, K_, generator=g), _bf(torch.randn(E, n, K_, generator=g))
    idx = torch.randint(0, E + 1, (M * top,), generator=g).to(torch.int32)
    idx[0], idx[1] = E, 0
    c = torch.full((M * top, n), 5.0, device="cuda")
    check(L.mn_gemv_f32_indexed_upto(ptr(D(a)), K_, top, ptr(D(w)), K_, n * K_, ptr(D(idx)), E, ptr(c), n, M * top, n, K_, stream()))
    for z in range(M * top):
        ref = torch.full((n,), 5.0, dtype=torch.float64) if idx[z] >= E else w[idx[z]].double() @ a[z // top].double()
        assert err(c[z], ref) < 1e-5
    x, base, h, add, tw = (torch.randn(s_, generator=g) for s_ in ((M, n), (M * top, n), (M, n), (M, n), (M, top)))
    slot_of = torch.randperm(M * top, generator=g).to(torch.int32)
    real = (idx < E).reshape(M, top)
    ref = x.double() + add.double() + (tw.double() * real)[:, :, None].mul(base.double().reshape(M, top, n)).sum(1) + \
        (tw.double() * ~real).sum(1, keepdim=True) * h.double()
    holes = base.clone()
    holes[idx >= E] = float("nan")                               # rows no product wrote are never read
    for so in (None, slot_of):
        ye = holes if so is None else torch.empty_like(holes).index_copy_(0, so.long(), holes)
        xd = x.cuda()
        check(L.mn_moe_combine_pass_residual(ptr(xd), n, ptr(D(ye)), n, ptr(D(so)) if so is not None else None, ptr(D(idx)), ptr(D(tw)), top, E,
                                             ptr(D(h)), n, ptr(D(add)), n, M, n, stream()))
        assert err(xd, ref) < 1e-6


# ---- whole models ------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", MODELS)
def test_prompt_layers_and_logits(name):
    cfg, sd, dec = make(name)
    t = toks(cfg, 81)                                     # above 64 rows: the recurrence runs as a chunked scan
    ref, streams = O.forward(cfg, sd, t, trace=True)
    hid, tr = dec.forward_spans(dec.embed(torch.tensor(t, device="cuda")), [(0, len(t), 0)], trace=True)
    assert tr.shape[0] == len(O.run_order(cfg))
    for r in range(tr.shape[0]):
        assert err(tr[r], streams[r]) < 1e-4, r
    assert err(dec.logits(hid), ref) < 1e-4


@pytest.mark.parametrize("name", ["mixed", "odd", "ones"])
def test_first_tokens(name):
    """The first positions: a recurrence from zero on a reused state, a softmax over one key and the sink, the temperature's first steps."""
    cfg, sd, dec = make(name)
    run_portions(dec, 0, toks(cfg, 9, 8), [9])            # leaves keys and a state behind
    t = toks(cfg, 6, 5)
    ref = O.forward(cfg, sd, t)
    assert err(run_portions(dec, 0, t, [1] * 6), ref) < 1e-4
    assert err(run_portions(dec, 0, t, [2, 2, 2]), ref) < 1e-4
    assert err(run_portions(dec, 0, t[:1], [1]), ref[:1]) < 1e-4


@pytest.mark.parametrize("name", MODELS)
def test_portions_and_decoding(name):
    cfg, sd, dec = make(name)
    t = toks(cfg, 150, 2)
    ref = O.forward(cfg, sd, t)
    assert err(run_portions(dec, 0, t, [110] + [1] * 40), ref) < 1e-4                      # prefill (scan) against token-by-token decoding
    assert err(run_portions(dec, 0, t, [7, 2, 13, 2, 2, 1, 19, 3, 2, 24, 70, 5]), ref) < 1e-4   # portions cut inside chunks and key tiles
    assert err(run_portions(dec, 0, t[:75], [1] * 75), ref[:75]) < 1e-4


def test_single_far_keys_decide_in_prompts_and_decoding():
    """Peaky attention, so that single keys — often far back — carry the result, in one piece, in portions and decoded one by one."""
    cfg, sd, dec = make("mixed", peaky=12.0, seed=7)
    t = toks(cfg, 140, 9)
    ref = O.forward(cfg, sd, t)
    assert err(run_portions(dec, 0, t, [140]), ref) < 2e-4
    assert err(run_portions(dec, 0, t, [80] + [1] * 60), ref) < 2e-4
    assert err(run_portions(dec, 0, t, [9, 3, 4, 5, 11, 2, 30, 66, 10]), ref) < 2e-4


def test_unequal_requests_share_a_pass():
    """Three requests of different lengths in one pass, then a pass that mixes a prompt portion of one with single decode rows of
    the others: every request's logits equal the oracle on that request alone."""
    cfg, sd, dec = make("mixed", n_seq=4)
    reqs = {3: toks(cfg, 120, 1), 0: toks(cfg, 9, 2), 2: toks(cfg, 43, 3)}
    refs = {s: O.forward(cfg, sd, t) for s, t in reqs.items()}
    first = {3: 70, 0: 8, 2: 42}
    ids = torch.tensor([x for s, t in reqs.items() for x in t[:first[s]]], device="cuda")
    lg = dec.logits(dec.forward_spans(dec.embed(ids), [(s, first[s], 0) for s in reqs]))
    r0 = 0
    for s in reqs:
        assert err(lg[r0:r0 + first[s]], refs[s][:first[s]]) < 1e-4
        r0 += first[s]
    ids = torch.tensor([reqs[0][8]] + reqs[3][70:120] + [reqs[2][42]], device="cuda")
    lg = dec.logits(dec.forward_spans(dec.embed(ids), [(0, 1, 8), (3, 50, 70), (2, 1, 42)]))
    assert err(lg[0:1], refs[0][8:9]) < 1e-4 and err(lg[1:51], refs[3][70:120]) < 1e-4 and err(lg[51:52], refs[2][42:43]) < 1e-4


def test_inputs_longer_than_a_pass(monkeypatch):
    """More rows than one pass through the stack takes: the passes cut a sequence inside a chunk and a key tile, and a later sequence
    starts inside a pass; the trace is stitched across passes."""
    from ming_univision_amd import seq_lm
    monkeypatch.setattr(seq_lm, "MAX_ROWS", 70)
    cfg, sd, dec = make("mixed", n_seq=2)
    a, b = toks(cfg, 160, 1), toks(cfg, 31, 2)
    (ra, sa), rb = O.forward(cfg, sd, a, trace=True), O.forward(cfg, sd, b)
    ids = torch.tensor(a + b, device="cuda")
    hid, tr = dec.forward_spans(dec.embed(ids), [(1, 160, 0), (0, 31, 0)], trace=True)
    lg = dec.logits(hid)
    assert err(lg[:160], ra) < 1e-4 and err(lg[160:], rb) < 1e-4 and err(tr[-1][:160], sa[-1]) < 1e-4
    with pytest.raises(AssertionError):
        dec.forward_spans(dec.embed(ids[:10]), [(0, 10, dec.t_max - 5)])       # beyond the cache: refused, not written


def test_released_sequences_are_reused():
    """A cache sequence that held a longer request is given back and reused: its old keys and recurrent states stay in memory and
    must not leak into the next request (nothing is cleared)."""
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
    dec.release_sequences(2)
    got = dec.logits(dec.forward_spans(dec.embed(torch.tensor(more, device="cuda")), [(a, 6, 36)]))        # a lives on after the shrink
    assert err(got, O.forward(cfg, sd, t + more + more)[36:]) < 1e-4


def test_long_decoding():
    cfg, sd, dec = make("odd")
    t = toks(cfg, 300, 11)
    got = run_portions(dec, 0, t, [5] + [1] * 295)
    assert err(got, O.forward(cfg, sd, t)) < 1e-4


def rows_off(got, want, tol):
    """-> (rows whose error is above tol of the logits' scale, median row error).  bf16-rounded router inputs may flip a close call
    between two experts, which changes single rows by more than rounding does; such rows are counted, not averaged away."""
    want = want.double()
    e = (got.double().cpu() - want).abs().amax(-1) / want.abs().max()
    return int((e > tol).sum()), float(e.median())


def test_bf16_arithmetic():
    """Serving arithmetic: portions above 64 rows take the bf16 MFMA products and the experts sorted on the grouped MFMA GEMMs (rows
    within 3e-2 of the logits' scale against the oracle, but for a few whose routing was a close call; median below 1e-2), portions
    of 9 .. 64 rows the weight-streaming MFMA route on hi/lo rows, rows fed a few at a time fp32 FMA."""
    for name in ("mixed", "odd", "wide", "tail"):         # "odd": no K is a multiple of 8; "wide": too many experts for the sorted route; "tail": the 256-tile grouped route
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
    """ZuzenexForCausalLM.generate: unequal prompts in one lock-step batch; every new token is the oracle's arg-max given the
    tokens before it (or the oracle's two best are within 1e-4), alone or batched, with and without the captured decode step;
    sampled generation returns tokens and gives its cache sequences back."""
    from ming_univision_amd.zuzenex import ZuzenexForCausalLM
    cfg, sd, dec = make("mixed")
    lm = ZuzenexForCausalLM(dec)
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
    synchronisations between replays, across a re-capture."""
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
    expert width multiples of 64), pass-through picks sorted behind them.  The captured step, replayed, picks the same tokens as the
    eager one, and the logits of the batch stay within the bf16 tolerance of the oracle."""
    from ming_univision_amd.zuzenex import ZuzenexForCausalLM
    cfg = O.small_config([O.lightning_layer(mlp=O.moe(5, 2, 64, identity=2, shared=64)), O.attention_layer(mlp=O.moe(3, 2, 128))], loop=(0, 1, 2))
    sd = O.random_weights(cfg, 5)
    dec = build(cfg, sd, arith="bf16", t_max=128, n_seq=10)
    lm = ZuzenexForCausalLM(dec)
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
