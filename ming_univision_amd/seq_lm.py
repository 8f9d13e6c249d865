"""What the decoder-only language models of this framework share: stepping rows of several cache sequences through a stack in
passes, the vocabulary projection and the picks, a decode step captured as a HIP graph, and the lock-step generation loop.

A decoder class (`pizitar.PizitarDecoder`, `sakinex.SakinexDecoder`, `zuzenex.ZuzenexDecoder`) owns its weights, caches and states and gives
    step(x, row_seq, row_slot, row_back, row_len, blk_tab, max_len, out, trace, ws, distinct)   one pass over <= max_rows() rows
    _workspace_bytes(rows, max_len), ensure_sequences(n), release_sequences(n), n_trace (residual streams a trace holds)
(a decoder with a `chunk_rows` attribute also gets chunk_tab = its rows cut into chunks of that many rows of one sequence; a decoder
whose layers read the token ids themselves sets `needs_tokens` and gets row_tok = the rows' ids as an int32 device array)
and inherits the rest from `SeqDecoder`; its generation entry point derives from `SeqCausalLM`.
"""
import ctypes as C

import numpy as np
import torch

from . import ops
from ._lib import check, current_stream, lib, ptr
from .sequences import SequenceSlots, rows_of_spans

MAX_ROWS = 2048          # rows of one pass through the stack; longer inputs run as several passes
ARITH = {"bf16": 0, "f32": 1}


class SeqDecoder:
    """Needs: cfg (width, optional logit_softcap), device, embed_w, head_w, arith, t_max, block_rows, n_trace, _ws, _decode_tabs."""

    def max_rows(self):
        return MAX_ROWS

    # ---- stepping -------------------------------------------------------------------------------------------------------------
    def _workspace(self, rows, max_len):
        key = torch.cuda.current_stream().cuda_stream
        need = int(self._workspace_bytes(rows, max_len))
        if key not in self._ws or self._ws[key].numel() < need:
            self._ws[key] = torch.empty(need, dtype=torch.uint8, device=self.device)
        return self._ws[key]

    needs_tokens = False

    def forward_spans(self, x, spans, trace=False, tokens=None):
        """Rows of several sequences through the stack: spans = [(cache sequence, rows, tokens it already holds)] in row order,
        x fp32 [sum rows, width]; tokens: the rows' ids (a decoder with `needs_tokens` reads them).  Runs in passes of <= max_rows()
        rows; a sequence cut by a pass boundary continues in the next pass.  Returns the final-norm hidden states [rows, width] (and
        the per-layer residual streams when trace)."""
        M = x.shape[0]
        assert sum(n for _, n, _ in spans) == M
        if self.needs_tokens:
            assert tokens is not None and tokens.numel() == M, "this decoder's layers read the token ids: pass tokens="
            tokens = tokens.reshape(-1).to(self.device, torch.int32).contiguous()
        out = torch.empty(M, self.cfg.width, dtype=torch.float32, device=self.device)
        tr = torch.empty(self.n_trace, M, self.cfg.width, dtype=torch.float32, device=self.device) if trace else None
        starts = np.cumsum([0] + [n for _, n, _ in spans])
        for r0 in range(0, M, self.max_rows()):
            r1 = min(M, r0 + self.max_rows())
            part = [(seq, min(starts[i + 1], r1) - max(starts[i], r0), past + max(starts[i], r0) - starts[i])
                    for i, (seq, n, past) in enumerate(spans) if min(starts[i + 1], r1) > max(starts[i], r0)]
            tabs = rows_of_spans([(int(s), int(n), int(p)) for s, n, p in part], self.block_rows, getattr(self, "chunk_rows", 0))
            dev = {k: torch.from_numpy(v).to(self.device) for k, v in tabs.items() if k != "max_len"}
            ptr_tr = None
            if trace:
                ptr_tr = torch.empty(self.n_trace, r1 - r0, self.cfg.width, dtype=torch.float32, device=self.device)
            self.step(x[r0:r1], dev["row_seq"], dev["row_slot"], dev["row_back"], dev["row_len"], dev["blk_tab"], tabs["max_len"],
                      out=out[r0:r1], trace=ptr_tr, distinct=all(n == 1 for _, n, _ in part),
                      **({"chunk_tab": dev["chunk_tab"]} if "chunk_tab" in dev else {}),
                      **({"row_tok": tokens[r0:r1]} if self.needs_tokens else {}))
            if trace:
                tr[:, r0:r1] = ptr_tr
        return (out, tr) if trace else out

    def prefill(self, ids, seq=0, past=0):
        """Tokens ids (int tensor [T]) of ONE sequence from slot `past`; returns the hidden states [T, width]."""
        return self.forward_spans(self.embed(ids), [(seq, int(ids.numel()), past)], tokens=ids)

    def decode_tables(self, B):
        """Static per-row tables of a lock-step decode step of B sequences (one row each): (row_back, blk_tab)."""
        if B not in self._decode_tabs:
            self._decode_tabs[B] = (torch.zeros(B, dtype=torch.int32, device=self.device),
                                    torch.stack([torch.arange(B, dtype=torch.int32), torch.ones(B, dtype=torch.int32)], 1).contiguous().to(self.device))
        return self._decode_tabs[B]

    def decode_graph(self, row_seq, row_slot, row_len):
        """A replayable lock-step decode step of B = len(row_seq) sequences (one row each): `DecodeGraph`."""
        return DecodeGraph(self, row_seq, row_slot, row_len)

    # ---- vocabulary -------------------------------------------------------------------------------------------------------------
    def embed(self, ids):
        return ops.bf16_to_f32(self.embed_w[ids.reshape(-1).to(self.device)])

    def logits(self, hidden):
        """Vocabulary projection + soft cap -> fp32 [M, vocab]."""
        hidden = hidden.contiguous()
        M, K = hidden.shape
        V = self.head_w.shape[0]
        out = torch.empty(M, V, dtype=torch.float32, device=self.device)
        ws = torch.empty(max(M * K * 2, 16), dtype=torch.uint8, device=self.device)
        check(lib().mn_seq_logits(ptr(hidden), K, M, ptr(self.head_w), V, K, float(getattr(self.cfg, "logit_softcap", None) or 0.0), ARITH[self.arith],
                                  ptr(out), V, ptr(ws), ws.numel(), current_stream()), "mn_seq_logits")
        return out

    def greedy(self, hidden):
        """Greedy pick of every row -> int64 [M] on the device.  The soft cap is increasing, so the arg-max of the uncapped
        product is the arg-max of the logits: the other decoder's fused vocabulary-projection + arg-max call serves here too
        (width a multiple of 8; otherwise through `logits`)."""
        if hidden.shape[1] % 8 == 0:
            return ops.lmhead_argmax(hidden.contiguous(), self.head_w)[0]
        return self.logits(hidden).argmax(-1)

    def sample(self, hidden, u, temperature=1.0, top_k=50, top_p=1.0):
        """Sampled pick of every row at the caller's uniforms u fp32 [M] (temperature -> top-k -> top-p -> one draw)."""
        return ops.sample_logits(self.logits(hidden), u, temperature, top_k, top_p)



class DecodeGraph:
    """One lock-step decode step (stack pass + advancing the rows' slots and lengths) captured as a HIP graph: a step of a small
    model is some twenty short launches per layer, and their host-side launch cost, not the kernels, bounds it.  The per-row
    state lives in device arrays that the graph's own last node advances, the input rows are copied into a fixed buffer, and the
    only host number baked in is an upper bound of the lengths (it sizes the attention's key splits), so one capture serves
    `span` tokens; `run` re-captures when the lengths pass the bound."""

    def __init__(self, dec, row_seq, row_slot, row_len, span=256):
        self.dec, self.span = dec, span
        self.row_seq, self.slot, self.len = row_seq, row_slot, row_len
        B = row_seq.numel()
        self.B = B
        self.back, self.blk = dec.decode_tables(B)
        self.x = torch.zeros(B, dec.cfg.width, dtype=torch.float32, device=dec.device)
        self.out = torch.empty(B, dec.cfg.width, dtype=torch.float32, device=dec.device)
        self.tok = torch.zeros(B, dtype=torch.int32, device=dec.device) if dec.needs_tokens else None
        n = int(dec._workspace_bytes(B, dec.t_max))
        self.ws = torch.empty(n, dtype=torch.uint8, device=dec.device)
        self.bound, self.graph = 0, None

    def _body(self):
        self.dec.step(self.x, self.row_seq, self.slot, self.back, self.len, self.blk, self.bound, out=self.out, ws=self.ws, distinct=True,
                      **({"row_tok": self.tok} if self.tok is not None else {}))
        check(lib().mn_rows_advance(ptr(self.slot), ptr(self.len), None, self.B, 1, current_stream()), "mn_rows_advance")

    def run(self, x, max_len, tokens=None):
        """x fp32 [B, width]: the new tokens' embeddings (tokens: their ids, for a decoder with `needs_tokens`); max_len: host upper
        bound of the lengths after this step.  Returns the hidden states [B, width] (a fixed buffer, overwritten by the next run)."""
        if self.tok is not None:
            self.tok.copy_(tokens.reshape(-1))
        if self.graph is None or max_len > self.bound:
            self.bound = min(self.dec.t_max, (max_len + self.span - 1) // self.span * self.span)
            self.graph = torch.cuda.CUDAGraph()
            self.x.copy_(x)
            torch.cuda.synchronize(self.dec.device)
            snap = (self.slot.clone(), self.len.clone())
            with torch.cuda.graph(self.graph):
                self._body()
            # capture records, it does not run: the arrays are untouched, but restore them in case a runtime ever executes eagerly
            self.slot.copy_(snap[0])
            self.len.copy_(snap[1])
        self.x.copy_(x)
        self.graph.replay()
        return self.out


class SeqCausalLM:
    """Generation entry point: requests in, token ids out, in lock-step batches (the batching of the other decoder's
    `generate_text_batch`): all prompts share the prefill passes, then one pass per new token serves every live sequence."""

    def __init__(self, decoder, eos_token_id=None):
        self.dec = decoder
        self.eos_token_id = eos_token_id
        self.slots = SequenceSlots(decoder)

    @torch.no_grad()
    def generate(self, prompts, max_new_tokens=16, do_sample=False, temperature=1.0, top_k=50, top_p=1.0, generator=None, sync_every=8,
                 use_graph=None):
        """prompts: list of token-id lists (unequal lengths allowed).  Greedy, or sampled (new token i of request b uses uniform
        [i, b] of one torch.rand(max_new_tokens, B) draw).  use_graph: run the decode steps as replays of a captured HIP graph
        (default: from 8 new tokens on).  Returns the new tokens of every request (cut after the first EOS)."""
        dec, dev = self.dec, self.dec.device
        B = len(prompts)
        lens = [len(p) for p in prompts]
        if min(lens) < 1 or max(lens) + max_new_tokens > dec.t_max:
            raise ValueError(f"prompts of 1 .. {dec.t_max - max_new_tokens} tokens (t_max = {dec.t_max})")
        seqs = [self.slots.alloc() for _ in range(B)]
        try:
            ids = torch.tensor([t for p in prompts for t in p], dtype=torch.long, device=dev)
            hid = dec.forward_spans(dec.embed(ids), [(s, n, 0) for s, n in zip(seqs, lens)], tokens=ids)
            last = torch.tensor(np.cumsum(lens) - 1, dtype=torch.long, device=dev)
            hidden = hid[last].contiguous()
            row_seq = torch.tensor(seqs, dtype=torch.int32, device=dev)
            slot = torch.tensor(lens, dtype=torch.int32, device=dev)
            ln = slot + 1
            back, blk = dec.decode_tables(B)
            graph = dec.decode_graph(row_seq, slot, ln) if (max_new_tokens >= 8 if use_graph is None else use_graph) else None
            finished = torch.zeros(B, dtype=torch.bool, device=dev)
            uniforms = torch.rand(max_new_tokens, B, device=dev, generator=generator) if do_sample else None
            toks = []
            for i in range(max_new_tokens):
                tok = dec.sample(hidden, uniforms[i], temperature, top_k, top_p) if do_sample else dec.greedy(hidden)
                toks.append(tok)
                if self.eos_token_id is not None:
                    finished |= tok == self.eos_token_id
                    if (i + 1) % sync_every == 0 and bool(finished.all()):
                        break
                if i + 1 == max_new_tokens:
                    break
                if graph is not None:
                    hidden = graph.run(dec.embed(tok), max(lens) + i + 1, tokens=tok)
                else:
                    hidden = dec.step(dec.embed(tok), row_seq, slot, back, ln, blk, max(lens) + i + 1, distinct=True,
                                      **({"row_tok": tok.to(torch.int32)} if dec.needs_tokens else {}))
                    check(lib().mn_rows_advance(ptr(slot), ptr(ln), None, B, 1, current_stream()), "mn_rows_advance")
            out = torch.stack(toks, 1).tolist()
        finally:
            for s in seqs:
                self.slots.release(s)
        res = []
        for row in out:
            if self.eos_token_id is not None and self.eos_token_id in row:
                row = row[:row.index(self.eos_token_id) + 1]
            res.append(row)
        return res
