"""Prefill / decode throughput of the Pizitar, the Sakinex or the Zuzenex decoder beside the Bailing-MoE decoder at equal size
(`bench.py --lm-compare [--lm-model sakinex | zuzenex]`), and of the Daberax decoder beside the Zuzenex decoder (`--lm-model daberax`).

Random weights at sizes that resemble real layers.  "Equal size": same width, depth and head count, 128-wide heads on both, and a
feed-forward whose ACTIVE hidden width matches (the MoE runs 8 experts, top-2, of half the dense hidden width each).  Both run
their serving paths: Pizitar `forward_spans` / `step` (bf16 arithmetic), Bailing-MoE `prefill_mfma` (its bf16 regime) and `step`.
Beside the end-to-end rates the attention kernels are timed alone against their rooflines — what each must move or multiply:
  decode   bytes of cache read per step / HBM peak        (latents [len, r] fp32  vs  keys + values [len, n_kv, 128] x 2 fp32)
  prefill  multiply-adds of the causal score / value products at the precision the kernel runs them
           (fp32 FMA peak for the latent kernel, bf16 MFMA peak for the flash kernel)

Sakinex at "equal size": same width, depth, query / key-value head counts and 128-wide heads as the Bailing-MoE side, the same 8
experts, top-2, plus one shared expert on both, a recurrence as wide as the model, a window of 1024 tokens with pooled blocks of 16,
no repeated layers.  Its attention reads at most window + length / pool keys per row, so its rooflines are priced on THOSE keys:
  decode   bytes of the visible keys and values (token arenas + block-mean arenas) per step / HBM peak
  prefill  multiply-adds of the visible score / value products on the fp32 FMA peak (the kernel's arithmetic)
and the recurrence alone on the bytes it reads and writes.

Zuzenex at "equal size": same width, depth, query / key-value head counts and 128-wide heads, layers attention - lightning - lightning -
attention, 8 experts top-2 plus one pass-through output and one shared expert (its experts have two matrices where the SwiGLU experts
have three, so they are 1.5 times as wide: the same parameters per expert).  Its attention sees every earlier token, like the other
decoder's, and is priced the same way — on the fp32 matrix-core peak for prompts (its scores and weights are 32-bit) and on the cache
bytes for decode rows; the recurrence alone is priced on its multiply-adds (prompts: the chunked scan) and on the state bytes it reads
and writes (decode rows).

Daberax stands beside Zuzenex, the closest model of the framework (both choose attention or a matrix-state recurrence per layer): same
width, depth, head counts and 128-wide heads, dense feed-forwards of equal parameter count on both (three matrices of width ff against
two of 1.5 ff), layers latent - delta - delta - attention against attention - lightning - lightning - attention.  Daberax's attentions
see a window of 1024 tokens and are priced on the keys they see; its latent attention reads [latent ; rotated part] once per key (the
values are a view of the keys); the delta rule is priced like the lightning recurrence — prompts on the multiply-adds of the recurrence
(three products of a dim x vdim state per token and head), decode rows on the state bytes read and written.
"""
import time

import torch

HBM_GBS = 8000.0
MFMA_BF16_TFLOPS = 2500.0
FMA_F32_TFLOPS = 157.3

SIZES = {
    "w1024": dict(width=1024, layers=4, heads=8, kv_rank=256, q_rank=384, ff=4096, vocab=32000),
    "w2048": dict(width=2048, layers=4, heads=16, kv_rank=512, q_rank=768, ff=8192, vocab=32000),
}


def _time(fn, iters, warm=2):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / iters


def pizitar_config(s):
    from .configuration import PizitarConfig
    la = dict(type="latent_attention", mixer=dict(heads=s["heads"], dim=128, vdim=128, kv_rank=s["kv_rank"], q_rank=s["q_rank"], scale=128 ** -0.5),
              mlp=dict(kind="dense", ff=s["ff"]))
    lb = dict(type="latent_attention_2", mixer=dict(heads=s["heads"], dim=128, vdim=128, kv_rank=s["kv_rank"], scale=128 ** -0.5),
              mlp=dict(kind="dense", ff=s["ff"]))
    return PizitarConfig(width=s["width"], vocab=s["vocab"], layers=[la, lb] * (s["layers"] // 2), canon=dict(taps=4), norm=dict(eps=1e-6),
                         logit_softcap=30.0)


def sakinex_config(s):
    from .configuration import SakinexConfig
    left = dict(conv=4, dim=128, vdim=128, heads=s["heads"], kv_heads=s["heads"] // 4, mask=dict(pool=SAKINEX_POOL, size=SAKINEX_WINDOW),
                rot=dict(base=600000.0, dims=128, scaling=dict(factor=4.0, fast=16.0, original=4096, slow=1.0)), scale=128 ** -0.5)
    ly = dict(type="parallel", mixer=dict(left=left, left_scale=0.7, right=dict(width=s["width"]), right_scale=0.7),
              mlp=dict(kind="moe", router=dict(experts=8, top=2), expert=dict(ff=s["ff"] // 2), shared=dict(ff=s["ff"] // 2)))
    return SakinexConfig(width=s["width"], vocab=s["vocab"], layers=[ly] * s["layers"], canon=dict(taps=4), norm=dict(eps=1e-6), residual_mult=0.5)


SAKINEX_WINDOW, SAKINEX_POOL = 1024, 16


def bailing_config(s, shared=0):
    from .configuration import BailingMoeConfig
    return BailingMoeConfig(vocab_size=s["vocab"], hidden_size=s["width"], num_hidden_layers=s["layers"], num_attention_heads=s["heads"],
                            num_key_value_heads=s["heads"] // 4, head_dim=128, use_bias=False, use_qkv_bias=False, rope_theta=600000.0,
                            num_experts=8, num_shared_experts=shared, num_experts_per_tok=2, moe_intermediate_size=s["ff"] // 2, multi_gate=False,
                            first_k_dense_replace=0, norm_topk_prob=True)


def run_pizitar(s, T, batches, n_dec):
    from ._lib import check, current_stream, lib, ptr
    from .pizitar import PizitarDecoder
    dev = "cuda"
    cfg = pizitar_config(s)
    dec = PizitarDecoder.synthetic(cfg, dev, t_max=T + n_dec + 8, n_seq=max(batches), arith="bf16")
    ids = torch.randint(0, s["vocab"], (T,), device=dev)
    x = dec.embed(ids)
    out = {"prefill_tokens_per_s": T / _time(lambda: dec.forward_spans(x, [(0, T, 0)]), 3)}
    for B in batches:
        for b in range(1, B):
            for a in dec.latent:
                a[b, :T] = a[0, :T]
            dec.taps_state[:, b] = dec.taps_state[:, 0]
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        back, blk = dec.decode_tables(B)
        xb = dec.embed(torch.randint(0, s["vocab"], (B,), device=dev))

        def loop():
            slot = torch.full((B,), T, dtype=torch.int32, device=dev)
            ln = slot + 1
            for i in range(n_dec):
                dec.step(xb, row_seq, slot, back, ln, blk, T + i + 1, distinct=True)
                check(lib().mn_rows_advance(ptr(slot), ptr(ln), None, B, 1, current_stream()), "mn_rows_advance")
        out[f"decode_b{B}_tokens_per_s"] = B * n_dec / _time(loop, 2, 1)
        slot_g = torch.full((B,), T, dtype=torch.int32, device=dev)
        ln_g = slot_g + 1
        graph = dec.decode_graph(row_seq, slot_g, ln_g)

        def loop_graph():
            slot_g.fill_(T)
            ln_g.fill_(T + 1)
            for i in range(n_dec):
                graph.run(xb, T + i + 1)
        out[f"decode_b{B}_graph_tokens_per_s"] = B * n_dec / _time(loop_graph, 2, 1)
    # the attention kernel alone
    H, r = s["heads"], s["kv_rank"]
    tabs = {k: (torch.from_numpy(v).to(dev) if k != "max_len" else v) for k, v in
            __import__("ming_univision_amd.sequences", fromlist=["x"]).rows_of_spans([(0, T, 0)], dec.block_rows).items()}
    q = torch.randn(T, H, r, device=dev) * 0.05
    lat = torch.empty_like(q)
    nb = tabs["blk_tab"].shape[0]
    ks = lib().mn_latent_attn_splits(nb, T, r)
    ws = torch.empty(max(16, lib().mn_latent_attn_workspace_bytes(T, H, r, ks)), dtype=torch.uint8, device=dev)
    t = _time(lambda: check(lib().mn_latent_attn(ptr(q), ptr(dec.latent[0]), ptr(tabs["row_seq"]), ptr(tabs["row_len"]), ptr(tabs["blk_tab"]), nb,
                                                 T, H, r, dec.t_max, T, ks, ptr(lat), ptr(ws), ws.numel(), current_stream())), 5)
    flops = 2 * 2 * H * r * T * (T + 1) / 2
    out["attn_prefill"] = dict(us=t * 1e6, tflops=flops / t / 1e12, of_peak=flops / t / 1e12 / FMA_F32_TFLOPS, peak="fp32 FMA")
    for B in batches:
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        ln = torch.full((B,), T, dtype=torch.int32, device=dev)
        _, blk = dec.decode_tables(B)
        ks = lib().mn_latent_attn_splits(B, T, r)
        ws = torch.empty(max(16, lib().mn_latent_attn_workspace_bytes(B, H, r, ks)), dtype=torch.uint8, device=dev)
        t = _time(lambda: check(lib().mn_latent_attn(ptr(q), ptr(dec.latent[0]), ptr(row_seq), ptr(ln), ptr(blk), B, B, H, r, dec.t_max, T, ks,
                                                     ptr(lat), ptr(ws), ws.numel(), current_stream())), 20)
        byts = B * T * r * 4
        out[f"attn_decode_b{B}"] = dict(us=t * 1e6, gbs=byts / t / 1e9, of_peak=byts / t / 1e9 / HBM_GBS, key_splits=ks)
    return out


def run_sakinex(s, T, batches, n_dec):
    from ._lib import check, current_stream, lib, ptr
    from .sakinex import SakinexDecoder
    from .sequences import rows_of_spans
    dev = "cuda"
    cfg = sakinex_config(s)
    dec = SakinexDecoder.synthetic(cfg, dev, t_max=T + n_dec + 8, n_seq=max(batches), arith="bf16")
    ids = torch.randint(0, s["vocab"], (T,), device=dev)
    x = dec.embed(ids)
    out = {"prefill_tokens_per_s": T / _time(lambda: dec.forward_spans(x, [(0, T, 0)]), 3)}
    for B in batches:
        for run in dec.state_t:                              # every sequence continues the prompt of sequence 0
            for k, t in run.items():
                if t is not None:
                    ax = dec.SEQ_AXIS[k]
                    t.narrow(ax, 1, B - 1).copy_(t.narrow(ax, 0, 1).expand_as(t.narrow(ax, 1, B - 1))) if B > 1 else None
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        back, blk = dec.decode_tables(B)
        xb = dec.embed(torch.randint(0, s["vocab"], (B,), device=dev))

        def loop():
            slot = torch.full((B,), T, dtype=torch.int32, device=dev)
            ln = slot + 1
            for i in range(n_dec):
                dec.step(xb, row_seq, slot, back, ln, blk, T + i + 1, distinct=True)
                check(lib().mn_rows_advance(ptr(slot), ptr(ln), None, B, 1, current_stream()), "mn_rows_advance")
        out[f"decode_b{B}_tokens_per_s"] = B * n_dec / _time(loop, 2, 1)
        slot_g = torch.full((B,), T, dtype=torch.int32, device=dev)
        ln_g = slot_g + 1
        graph = dec.decode_graph(row_seq, slot_g, ln_g)

        def loop_graph():
            slot_g.fill_(T)
            ln_g.fill_(T + 1)
            for i in range(n_dec):
                graph.run(xb, T + i + 1)
        out[f"decode_b{B}_graph_tokens_per_s"] = B * n_dec / _time(loop_graph, 2, 1)
    # the attention kernel alone, on the first run's arenas
    H, G, d = s["heads"], s["heads"] // 4, 128
    st = dec.state_t[0]
    tabs = {k: torch.from_numpy(v).to(dev) for k, v in rows_of_spans([(0, T, 0)], 1 << 30).items() if k != "max_len"}
    q = torch.randn(T, H * d, device=dev) * 0.05
    att = torch.empty(T, H * d, device=dev)

    RB = lib().mn_window_attn_block_rows()
    blk = torch.from_numpy(rows_of_spans([(0, T, 0)], RB)["blk_tab"]).to(dev)
    aws = torch.empty(64 << 20, dtype=torch.uint8, device=dev)

    def attn(M, rs, rp, one_row):
        n_blk = M if one_row else blk.shape[0]
        keys = SAKINEX_WINDOW + (0 if one_row else RB - 1) + T // SAKINEX_POOL
        ns = lib().mn_window_attn_splits(n_blk, H, G, one_row, keys)
        check(lib().mn_window_pool_attn_blocks(ptr(q), H * d, ptr(st["k"]), ptr(st["v"]), ptr(st["pk"]), ptr(st["pv"]), ptr(rs), ptr(rp),
                                               None if one_row else ptr(blk), n_blk, one_row, H, G, d, d, dec.t_max, dec.n_pool_max, SAKINEX_WINDOW,
                                               SAKINEX_POOL, 1.0, ptr(att), H * d, None, 0, ns, ptr(aws), aws.numel(), current_stream()),
              "mn_window_pool_attn_blocks")
        return ns

    def keys_at(i):
        return min(i + 1, SAKINEX_WINDOW) + max(0, (i - SAKINEX_WINDOW + 1) // SAKINEX_POOL)
    t = _time(lambda: attn(T, tabs["row_seq"], tabs["row_slot"], 0), 5)
    flops = 2 * 2 * H * d * sum(keys_at(i) for i in range(T))
    out["attn_prefill"] = dict(us=t * 1e6, tflops=flops / t / 1e12, of_peak=flops / t / 1e12 / FMA_F32_TFLOPS, peak="fp32 FMA")
    for B in batches:
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        slot = torch.full((B,), T - 1, dtype=torch.int32, device=dev)
        t = _time(lambda: attn(B, row_seq, slot, 1), 20)
        byts = B * keys_at(T - 1) * G * 2 * d * 4
        out[f"attn_decode_b{B}"] = dict(us=t * 1e6, gbs=byts / t / 1e9, of_peak=byts / t / 1e9 / HBM_GBS, keys=keys_at(T - 1),
                                        key_splits=attn(B, row_seq, slot, 1))
    # the recurrence alone: reads z, u, g, writes the gated state (fp32 rows)
    n = s["width"]
    zx, gg, o = torch.randn(T, 2 * n, device=dev), torch.randn(T, n, device=dev), torch.empty(T, n, device=dev)
    gws = torch.empty(lib().mn_mingru_scan_workspace_bytes(T, n), dtype=torch.uint8, device=dev)
    t = _time(lambda: check(lib().mn_mingru_rows_scan(ptr(zx), 2 * n, ptr(gg), n, ptr(st["gru"]), ptr(tabs["row_seq"]), ptr(tabs["row_slot"]),
                                                      ptr(tabs["row_back"]), 1.0, ptr(o), n, None, 0, T, n, ptr(gws), gws.numel(), current_stream()),
                            "mn_mingru_rows_scan"), 5)
    out["mingru_prefill"] = dict(us=t * 1e6, gbs=T * n * 16 / t / 1e9, of_peak=T * n * 16 / t / 1e9 / HBM_GBS)
    return out


def zuzenex_config(s, dense=False):
    from .configuration import ZuzenexConfig
    H = s["heads"]
    mlp = dict(kind="moe", router=dict(experts=8, top=2, identity=1), expert=dict(ff=s["ff"] * 3 // 4), shared=dict(ff=s["ff"] * 3 // 4))
    if dense:
        mlp = dict(kind="dense", ff=s["ff"] * 3 // 2)
    att = dict(type="attention", mixer=dict(heads=H, kv_heads=H // 4, dim=128, vdim=128, scale=128 ** -0.5, q_temp=dict(coef=0.1, every=1024)), mlp=mlp)
    lin = dict(type="lightning", mixer=dict(heads=H, dim=128, vdim=128, decay=[1.0 - 2.0 ** (-5 - 4 * h / H) for h in range(H)]), mlp=mlp)
    order = [att, lin, lin, att]
    return ZuzenexConfig(width=s["width"], vocab=s["vocab"], layers=[order[i % 4] for i in range(s["layers"])], norm=dict(eps=1e-6))


def run_zuzenex(s, T, batches, n_dec, dense=False):
    from ._lib import check, current_stream, lib, ptr
    from .sequences import rows_of_spans
    from .zuzenex import ZuzenexDecoder
    dev = "cuda"
    cfg = zuzenex_config(s, dense)
    dec = ZuzenexDecoder.synthetic(cfg, dev, t_max=T + n_dec + 8, n_seq=max(batches), arith="bf16")
    ids = torch.randint(0, s["vocab"], (T,), device=dev)
    x = dec.embed(ids)
    out = {"prefill_tokens_per_s": T / _time(lambda: dec.forward_spans(x, [(0, T, 0)]), 3)}
    for B in batches:
        for run in dec.state_t:                              # every sequence continues the prompt of sequence 0
            for t in run.values():
                if t is not None and B > 1:
                    t[1:B].copy_(t[0:1].expand_as(t[1:B]))
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        back, blk = dec.decode_tables(B)
        xb = dec.embed(torch.randint(0, s["vocab"], (B,), device=dev))

        def loop():
            slot = torch.full((B,), T, dtype=torch.int32, device=dev)
            ln = slot + 1
            for i in range(n_dec):
                dec.step(xb, row_seq, slot, back, ln, blk, T + i + 1, distinct=True)
                check(lib().mn_rows_advance(ptr(slot), ptr(ln), None, B, 1, current_stream()), "mn_rows_advance")
        out[f"decode_b{B}_tokens_per_s"] = B * n_dec / _time(loop, 2, 1)
        slot_g = torch.full((B,), T, dtype=torch.int32, device=dev)
        ln_g = slot_g + 1
        graph = dec.decode_graph(row_seq, slot_g, ln_g)

        def loop_graph():
            slot_g.fill_(T)
            ln_g.fill_(T + 1)
            for i in range(n_dec):
                graph.run(xb, T + i + 1)
        out[f"decode_b{B}_graph_tokens_per_s"] = B * n_dec / _time(loop_graph, 2, 1)
    # the attention kernel alone, on the first run's arenas (an attention layer)
    H, G, d = s["heads"], s["heads"] // 4, 128
    st = dec.state_t[0]
    RB = lib().mn_window_attn_block_rows()
    tabs = {k: torch.from_numpy(v).to(dev) for k, v in rows_of_spans([(0, T, 0)], RB, dec.chunk_rows).items() if k != "max_len"}
    q = torch.randn(T, H * d, device=dev) * 0.05
    att = torch.empty(T, H * d, device=dev)
    sink = torch.zeros(H, device=dev)
    aws = torch.empty(64 << 20, dtype=torch.uint8, device=dev)

    def attn(M, rs, rp, one_row):
        n_blk = M if one_row else tabs["blk_tab"].shape[0]
        ns = lib().mn_window_attn_splits(n_blk, H, G, one_row, T)
        check(lib().mn_window_pool_attn_blocks_sink(ptr(q), H * d, ptr(st["k"]), ptr(st["v"]), None, None, ptr(sink), ptr(rs), ptr(rp),
                                                    None if one_row else ptr(tabs["blk_tab"]), n_blk, one_row, H, G, d, d, dec.t_max, 1, 0, 0, 1.0,
                                                    ptr(att), H * d, None, 0, ns, ptr(aws), aws.numel(), -1, current_stream()),
              "mn_window_pool_attn_blocks_sink")
        return ns
    t = _time(lambda: attn(T, tabs["row_seq"], tabs["row_slot"], 0), 5)
    flops = 2 * 2 * H * d * T * (T + 1) / 2
    out["attn_prefill"] = dict(us=t * 1e6, tflops=flops / t / 1e12, of_peak=flops / t / 1e12 / FMA_F32_TFLOPS, peak="fp32 MFMA")
    for B in batches:
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        slot = torch.full((B,), T - 1, dtype=torch.int32, device=dev)
        t = _time(lambda: attn(B, row_seq, slot, 1), 20)
        byts = B * T * G * 2 * d * 4
        out[f"attn_decode_b{B}"] = dict(us=t * 1e6, gbs=byts / t / 1e9, of_peak=byts / t / 1e9 / HBM_GBS, key_splits=attn(B, row_seq, slot, 1))
    # the recurrence alone, on the second run's state (a lightning layer)
    lin = dec.state_t[1]["lin"]
    decay = torch.full((H,), 0.99, device=dev)
    qkv, o = torch.randn(T, 3 * H * d, device=dev), torch.empty(T, H * d, device=dev)
    n_ch = tabs["chunk_tab"].shape[0]
    sws = torch.empty(lib().mn_lightning_scan_workspace_bytes(n_ch, H, d, d), dtype=torch.uint8, device=dev)
    t = _time(lambda: check(lib().mn_lightning_rows_scan(ptr(qkv), 3 * H * d, T, H, d, d, ptr(decay), ptr(lin), ptr(tabs["row_seq"]), ptr(tabs["row_slot"]),
                                                         ptr(tabs["row_back"]), ptr(tabs["chunk_tab"]), n_ch, ptr(o), H * d, ptr(sws), sws.numel(),
                                                         current_stream()), "mn_lightning_rows_scan"), 5)
    C = dec.chunk_rows
    flops = 2 * T * H * (2 * d * d + C * 2 * d)             # per token and head: its k v^T, q against the carried state, the chunk's own scores and values
    out["lightning_prefill"] = dict(us=t * 1e6, tflops=flops / t / 1e12, of_peak=flops / t / 1e12 / FMA_F32_TFLOPS, peak="fp32 FMA")
    for B in batches:
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        slot = torch.full((B,), T - 1, dtype=torch.int32, device=dev)
        t = _time(lambda: check(lib().mn_lightning_rows(ptr(qkv), 3 * H * d, B, H, d, d, ptr(decay), ptr(lin), ptr(row_seq), ptr(slot), None, 1, ptr(o),
                                                        H * d, current_stream()), "mn_lightning_rows"), 20)
        byts = B * H * d * d * 4 * 2
        out[f"lightning_decode_b{B}"] = dict(us=t * 1e6, gbs=byts / t / 1e9, of_peak=byts / t / 1e9 / HBM_GBS)
    return out


def daberax_config(s, window=1024):
    from .configuration import DaberaxConfig
    H = s["heads"]
    mlp = dict(kind="dense", ff=s["ff"])
    att = dict(type="attention", mixer=dict(heads=H, kv_heads=H // 4, dim=128, vdim=128, scale=128 ** -0.5, softcap=50.0, mask=dict(size=window),
                                            rot=dict(base=1000000.0, dims=128, scaling=dict(factor=8.0, low=1.0, high=4.0, original=8192))), mlp=mlp)
    lat = dict(type="latent_attention", mixer=dict(heads=H, dim=128, rot_dim=64, vdim=128, kv_rank=s["kv_rank"], scale=192 ** -0.5,
                                                   mask=dict(size=window), rot=dict(base=10000.0, dims=64)), mlp=mlp)
    dlt = dict(type="delta", mixer=dict(heads=H, kv_heads=H // 2, dim=128, vdim=128, conv=4), mlp=mlp)
    order = [lat, dlt, dlt, att]
    return DaberaxConfig(width=s["width"], vocab=s["vocab"], layers=[order[i % 4] for i in range(s["layers"])], norm=dict(eps=1e-6),
                         token_side=dict(dim=64), logit_scale=0.5)


def run_daberax(s, T, batches, n_dec, window=1024):
    from ._lib import check, current_stream, lib, ptr
    from .daberax import DaberaxDecoder
    from .sequences import rows_of_spans
    dev = "cuda"
    cfg = daberax_config(s, window)
    dec = DaberaxDecoder.synthetic(cfg, dev, t_max=T + n_dec + 8, n_seq=max(batches), arith="bf16")
    ids = torch.randint(0, s["vocab"], (T,), device=dev)
    x = dec.embed(ids)
    out = {"prefill_tokens_per_s": T / _time(lambda: dec.forward_spans(x, [(0, T, 0)], tokens=ids), 3)}
    for B in batches:
        for ly in dec.state_t:                               # every sequence continues the prompt of sequence 0
            for t in ly.values():
                if t is not None and B > 1:
                    t[1:B].copy_(t[0:1].expand_as(t[1:B]))
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        back, blk = dec.decode_tables(B)
        tok = torch.randint(0, s["vocab"], (B,), device=dev)
        xb, tok32 = dec.embed(tok), tok.to(torch.int32)

        def loop():
            slot = torch.full((B,), T, dtype=torch.int32, device=dev)
            ln = slot + 1
            for i in range(n_dec):
                dec.step(xb, row_seq, slot, back, ln, blk, T + i + 1, distinct=True, row_tok=tok32)
                check(lib().mn_rows_advance(ptr(slot), ptr(ln), None, B, 1, current_stream()), "mn_rows_advance")
        out[f"decode_b{B}_tokens_per_s"] = B * n_dec / _time(loop, 2, 1)
        slot_g = torch.full((B,), T, dtype=torch.int32, device=dev)
        ln_g = slot_g + 1
        graph = dec.decode_graph(row_seq, slot_g, ln_g)

        def loop_graph():
            slot_g.fill_(T)
            ln_g.fill_(T + 1)
            for i in range(n_dec):
                graph.run(xb, T + i + 1, tokens=tok32)
        out[f"decode_b{B}_graph_tokens_per_s"] = B * n_dec / _time(loop_graph, 2, 1)
    # the kernels alone, on the layers' own arenas and states
    H = s["heads"]
    RB = lib().mn_window_attn_block_rows()
    tabs = {k: torch.from_numpy(v).to(dev) for k, v in rows_of_spans([(0, T, 0)], RB).items() if k != "max_len"}
    aws = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    pairs = sum(min(i + 1, window) for i in range(T))       # (query, key) pairs a prompt of T rows sees
    seen = min(T, window)

    def attention(name, li, G, dk, dv, ldk, v_of_k):
        st = dec.state_t[li]
        q = torch.randn(T, H * dk, device=dev) * 0.05
        att = torch.empty(T, H * dv, device=dev)
        varena = st["k"] if v_of_k else st["v"]

        def attn(M, rs, rp, one_row):
            n_blk = M if one_row else tabs["blk_tab"].shape[0]
            ns = lib().mn_window_attn_splits_tile(n_blk, H, G, one_row, seen, 16 if (v_of_k and one_row) else 64)
            check(lib().mn_window_pool_attn_blocks_cap(ptr(q), H * dk, ptr(st["k"]), ldk, ptr(varena), ldk if v_of_k else 0, None, None, None, 50.0,
                                                       ptr(rs), ptr(rp), None if one_row else ptr(tabs["blk_tab"]), n_blk, one_row, H, G, dk, dv,
                                                       dec.t_max, 1, window, 0, 1.0, ptr(att), H * dv, None, 0, ns, ptr(aws), aws.numel(), -1,
                                                       current_stream()), "mn_window_pool_attn_blocks_cap")
            return ns
        t = _time(lambda: attn(T, tabs["row_seq"], tabs["row_slot"], 0), 5)
        flops = 2 * H * (dk + dv) * pairs
        out[name + "_prefill"] = dict(us=t * 1e6, tflops=flops / t / 1e12, of_peak=flops / t / 1e12 / FMA_F32_TFLOPS,
                                      peak="fp32 MFMA" if max(dk, dv) <= 256 else "fp32 FMA")
        for B in batches:
            row_seq = torch.arange(B, dtype=torch.int32, device=dev)
            slot = torch.full((B,), T - 1, dtype=torch.int32, device=dev)
            t = _time(lambda: attn(B, row_seq, slot, 1), 20)
            byts = B * seen * (ldk if v_of_k else G * (dk + dv)) * 4
            out[f"{name}_decode_b{B}"] = dict(us=t * 1e6, gbs=byts / t / 1e9, of_peak=byts / t / 1e9 / HBM_GBS, key_splits=attn(B, row_seq, slot, 1))
    R = s["kv_rank"]
    attention("latent_attn", 0, 1, R + 64, R, lib().mn_pn_latent_ld(R, 64), True)
    attention("attn", 3, H // 4, 128, 128, 0, False)
    # the delta rule alone, on the second layer's state
    d, G = 128, H // 2
    lin = dec.state_t[1]["lin"]
    qkv = torch.randn(T, 2 * G * d + H * d, device=dev)
    qkv[:, :2 * G * d] *= d ** -0.5
    bd = torch.cat([torch.rand(T, H, device=dev), 0.9 + 0.1 * torch.rand(T, H, device=dev)], 1).contiguous()
    o = torch.empty(T, H * d, device=dev)

    def delta(M, rs, rp, rb, flags):
        check(lib().mn_gated_delta_rows(ptr(qkv), qkv.shape[1], ptr(bd), 2 * H, M, H, G, d, d, ptr(lin), ptr(rs), ptr(rp), ptr(rb), flags, ptr(o),
                                        H * d, current_stream()), "mn_gated_delta_rows")
    t = _time(lambda: delta(T, tabs["row_seq"], tabs["row_slot"], tabs["row_back"], 0), 5)
    flops = 2 * T * H * 3 * d * d
    out["delta_prefill"] = dict(us=t * 1e6, tflops=flops / t / 1e12, of_peak=flops / t / 1e12 / FMA_F32_TFLOPS, peak="fp32 FMA")
    for B in batches:
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        slot = torch.full((B,), T - 1, dtype=torch.int32, device=dev)
        back = torch.zeros(B, dtype=torch.int32, device=dev)
        t = _time(lambda: delta(B, row_seq, slot, back, 1), 20)
        byts = B * H * d * d * 4 * 2
        out[f"delta_decode_b{B}"] = dict(us=t * 1e6, gbs=byts / t / 1e9, of_peak=byts / t / 1e9 / HBM_GBS)
    return out


def run_bailing(s, T, batches, n_dec, shared=0):
    from . import ops
    from ._lib import check, current_stream, lib, ptr
    from .bailing_moe import BailingMoeDecoder
    dev = "cuda"
    cfg = bailing_config(s, shared)
    dec = BailingMoeDecoder.synthetic(cfg, dev, t_max=T + n_dec + 8, n_seq=max(batches))
    ids = torch.randint(0, s["vocab"], (T,), device=dev)
    x = dec.embed(ids)
    out = {"prefill_tokens_per_s": T / _time(lambda: dec.prefill_mfma(x, seq=0), 3),
           "prefill_fp32class_tokens_per_s": T / _time(lambda: dec.prefill_wide(x, seq=0), 3)}
    for B in batches:
        for b in range(1, B):
            dec.copy_sequence(0, b, T)
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        xb = dec.embed(torch.randint(0, s["vocab"], (B,), device=dev))

        def loop():
            slot = torch.full((B,), T, dtype=torch.int32, device=dev)
            ln = slot + 1
            for i in range(n_dec):
                dec.step(xb, row_seq, slot, slot, ln, distinct_sequences=True)
                check(lib().mn_rows_advance(ptr(slot), ptr(ln), None, B, 1, current_stream()), "mn_rows_advance")
        out[f"decode_b{B}_tokens_per_s"] = B * n_dec / _time(loop, 2, 1)
    nq, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, 128
    kv = dec.kv_cache[0]
    for B in batches:
        q = torch.randn(B, nq * hd, device=dev) * 0.05
        row_seq = torch.arange(B, dtype=torch.int32, device=dev)
        ln = torch.full((B,), T, dtype=torch.int32, device=dev)
        t = _time(lambda: ops.attn_decode(q, nq, nkv, hd, kv, row_seq, ln), 20)
        byts = B * T * nkv * hd * 2 * 4
        out[f"attn_decode_b{B}"] = dict(us=t * 1e6, gbs=byts / t / 1e9, of_peak=byts / t / 1e9 / HBM_GBS)
    # flash prefill alone (bf16 queries against the fp32 arena), one span of T rows
    qb = (torch.randn(T, nq * hd, device=dev) * 0.05).to(torch.bfloat16)
    att = torch.empty_like(qb)
    tab = torch.tensor([[0, 0, T]], dtype=torch.int32, device=dev)
    t = _time(lambda: check(lib().mn_flash_prefill_gqa_hd128(ptr(qb), ptr(kv), dec.t_max, nq, nkv, 0, ptr(tab), 1, T, None, 0, ptr(att),
                                                             current_stream())), 5)
    flops = 2 * 2 * nq * hd * T * (T + 1) / 2
    out["attn_prefill"] = dict(us=t * 1e6, tflops=flops / t / 1e12, of_peak=flops / t / 1e12 / MFMA_BF16_TFLOPS, peak="bf16 MFMA")
    return out


def compare(sizes=("w1024", "w2048"), prompt=2048, batches=(1, 32), n_dec=32, model="pizitar"):
    res = {}
    for name in sizes:
        s = SIZES[name]
        torch.cuda.empty_cache()
        if model == "daberax":                               # beside the closest model of the framework instead of the Bailing-MoE decoder
            res[name] = dict(size=s, prompt=prompt, daberax=run_daberax(s, prompt, batches, n_dec))
            torch.cuda.empty_cache()
            res[name]["zuzenex_dense"] = run_zuzenex(s, prompt, batches, n_dec, dense=True)
            continue
        if model == "zuzenex":
            res[name] = dict(size=s, prompt=prompt, zuzenex=run_zuzenex(s, prompt, batches, n_dec))
        elif model == "sakinex":
            res[name] = dict(size=s, prompt=prompt, sakinex=run_sakinex(s, prompt, batches, n_dec))
        else:
            res[name] = dict(size=s, prompt=prompt, pizitar=run_pizitar(s, prompt, batches, n_dec))
        torch.cuda.empty_cache()
        res[name]["bailing_moe"] = run_bailing(s, prompt, batches, n_dec, shared=1 if model in ("sakinex", "zuzenex") else 0)
    return res
