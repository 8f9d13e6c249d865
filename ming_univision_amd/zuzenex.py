"""Zuzenex: a decoder-only language model of hybrid-mixer layers, served by libmingnative's hybrid-mixer step function
(mingnative.h section 11: mn_hyb_step).

Per layer run, with x the fp32 residual stream of a token:
    h = RMS(x) w                                   one norm; the mixer and the feed-forward both read it
    x += mixer(h) + ff(h)
    mixer "attention": q, k, v = W h; q and k RMS-normed per head with a weight; q at position p times
                       1 + coef ln(floor((p + 1) / every) + 1); scores q . k * scale over every earlier token and itself; softmax whose
                       denominator also holds exp(sink_head); W_o on the heads
    mixer "lightning": q, k, v = silu(W h); per head S <- decay S + k v^T, o = S^T q (fp32 state per sequence); the joined heads
                       RMS-normed with a weight, times sigmoid(W_g h); W_o
    ff dense:          W_down relu(W_up h)^2
    ff moe:            s = softmax(W_r h) over all router outputs; the `top` largest of s + correction; weights = their s over their sum;
                       the last `identity` outputs stand for h itself; plus an always-on shared expert
A range of layers may run several times with the same weights (`loop`): every run has its own cache or state.  Then RMS and the
vocabulary projection.

This module owns HBM residency, like the other decoders' modules:
  * weights bf16; everything that reads h is stacked at load into ONE matrix [q ; k ; v ; (gate) ; up ; router] and the mixer's output
    projection is joined with the dense / shared expert's down projection along their inputs, so a layer is two dense products plus
    its experts, which lie in [experts, ff, width] / [experts, width, ff] blocks; sinks, decays and router corrections as fp32;
  * per layer RUN: fp32 key / value arenas [n_seq, t_max, .] (attention) or the fp32 recurrent state [n_seq, heads, dim, vdim]
    (lightning); cache sequences are numbered as in the other decoders (`sequences.SequenceSlots`); a number that is given back is
    reused as it is: a row at position 0 reads no state;
  * per-row int32 bookkeeping on the device, so a lock-step decode loop never syncs with the host.
`arith`: "bf16" = matrix products of steps above 8 rows on the bf16 MFMA kernels (fp32 accumulate), everything else fp32;
"f32" = fp32 FMA everywhere.
"""
import ctypes as C
import glob
import os

import torch

from . import _lib
from ._lib import HybLayer, HybModel, HybState, check, current_stream, lib, ptr
from .configuration import ZuzenexConfig, zuzenex_param_shapes
from .seq_lm import ARITH, SeqCausalLM, SeqDecoder

KIND = {"attention": 0, "lightning": 1}
FF_NONE, FF_DENSE, FF_MOE = 0, 1, 2


class ZuzenexDecoder(SeqDecoder):
    """Weights + per-run caches and states + the C-ABI tables of the stack."""

    def __init__(self, cfg: ZuzenexConfig, sd, t_max=2048, n_seq=1, arith="bf16"):
        """sd: {checkpoint tensor name: bf16 CUDA tensor}."""
        assert arith in ARITH, f"arith={arith!r}: 'bf16' or 'f32'"
        self.cfg, self.arith = cfg, arith
        missing = [k for k, shp in zuzenex_param_shapes(cfg).items() if k not in sd or tuple(sd[k].shape) != tuple(shp)]
        if missing:
            raise ValueError(f"checkpoint does not fit the configuration: missing or mis-shaped tensors {missing[:8]}")
        dev = sd["embed"].device
        self.device = dev
        self.embed_w, self.head_w = sd["embed"].contiguous(), sd["head"].contiguous()
        self.t_max, self.n_seq = int(t_max), int(n_seq)
        W = cfg.width
        self._keep = []                                  # packed tensors the C tables point to
        bf = dict(dtype=torch.bfloat16, device=dev)
        layers = (HybLayer * len(cfg.layers))()
        self.dims = []                                   # per layer: (kind, key channels, value channels, heads, dim, vdim)
        for i, ly in enumerate(cfg.layers):
            m, mlp, p, L = ly["mixer"], ly.get("mlp"), f"l{i}.", layers[i]
            H, d, e = int(m["heads"]), int(m["dim"]), int(m["vdim"])
            L.kind, L.heads, L.dim, L.vdim = KIND[ly["type"]], H, d, e
            L.norm1 = self._p(sd[p + "norm1"])
            stack = [sd[p + "mix.q"], sd[p + "mix.k"], sd[p + "mix.v"]]
            if ly["type"] == "attention":
                G = int(m["kv_heads"])
                L.kv_heads, L.scale = G, float(m["scale"])
                qt = m.get("q_temp")
                L.temp_every, L.temp_coef = (int(qt["every"]), float(qt["coef"])) if qt else (0, 0.0)
                L.q_norm, L.k_norm = self._p(sd[p + "mix.q.norm"]), self._p(sd[p + "mix.k.norm"])
                L.sink = self._f(sd[p + "mix.sink"].float())
            else:
                G = H
                L.kv_heads = H
                L.decay = self._f(torch.tensor([float(a) for a in m["decay"]], dtype=torch.float32, device=dev))
                L.mix_norm = self._p(sd[p + "mix.norm"])
                stack.append(sd[p + "mix.g"])
            out = [sd[p + "mix.o"]]
            L.ff_kind = FF_NONE
            if mlp is not None and mlp["kind"] == "dense":
                L.ff_kind, L.ff = FF_DENSE, int(mlp["ff"])
                stack.append(sd[p + "mlp.up"])
                out.append(sd[p + "mlp.down"])
            elif mlp is not None:
                r, q = mlp["router"], p + "mlp."
                E, ff = int(r["experts"]), int(mlp["expert"]["ff"])
                L.ff_kind, L.experts, L.n_pass, L.top, L.expert_ff = FF_MOE, E, int(r.get("identity") or 0), int(r["top"]), ff
                L.ff = int(mlp["shared"]["ff"]) if mlp.get("shared") else 0
                if L.ff:
                    stack.append(sd[q + "shared.up"])
                    out.append(sd[q + "shared.down"])
                stack.append(sd[q + "router"])
                L.correction = self._f(sd[q + "correction"].float())
                L.w_up = self._p(torch.stack([sd[f"{q}e{j}.up"] for j in range(E)]))
                L.w_down = self._p(torch.stack([sd[f"{q}e{j}.down"] for j in range(E)]))
            rows = sum(t.shape[0] for t in stack)
            stack.append(torch.zeros(-rows % 8, W, **bf))            # zero rows: the stack's row count a multiple of 8
            L.w_in = self._p(torch.cat(stack, 0))
            L.w_out = self._p(torch.cat(out, 1))
            self.dims.append((ly["type"], G * d, G * e, H, d, e))
        self._layers = layers
        runs = cfg.runs()
        self.runs = runs
        self.n_trace = len(runs)
        self._run_layer = (C.c_int32 * len(runs))(*runs)
        s = HybModel()
        s.width, s.n_layers, s.n_runs, s.arith, s.eps = W, len(cfg.layers), len(runs), ARITH[arith], cfg.eps
        s.layers = C.cast(layers, C.POINTER(HybLayer))
        s.run_layer = self._run_layer
        s.final_w = self._p(sd["final.norm"])
        self.struct = s
        self.state_t = self._alloc_state(self.n_seq)
        self._bind_state()
        self.block_rows = int(lib().mn_window_attn_block_rows())
        self.chunk_rows = int(lib().mn_lightning_chunk_rows())
        self._ws, self._decode_tabs = {}, {}

    def _p(self, t):
        assert t.dtype == torch.bfloat16 and t.is_cuda
        t = t.contiguous()
        self._keep.append(t)
        return t.data_ptr()

    def _f(self, t):
        assert t.dtype == torch.float32 and t.is_cuda
        t = t.contiguous()
        self._keep.append(t)
        return t.data_ptr()

    # ---- caches and states ---------------------------------------------------------------------------------------------------
    STATE_KEYS = ("k", "v", "lin")

    def _state_shapes(self, n_seq):
        """Per run: {name: shape or None}."""
        out = []
        for li in self.runs:
            kind, ck, cv, H, d, e = self.dims[li]
            attn = kind == "attention"
            out.append({"k": (n_seq, self.t_max, ck) if attn else None, "v": (n_seq, self.t_max, cv) if attn else None,
                        "lin": None if attn else (n_seq, H, d, e)})
        return out

    def _alloc_state(self, n_seq):
        return [{k: (None if shp is None else torch.zeros(shp, dtype=torch.float32, device=self.device)) for k, shp in run.items()}
                for run in self._state_shapes(n_seq)]

    def state_bytes_per_sequence(self):
        return sum(4 * int(torch.Size(shp).numel()) for run in self._state_shapes(1) for shp in run.values() if shp is not None)

    def _bind_state(self):
        self._tabs = {k: _lib.ptr_array([run[k] for run in self.state_t]) for k in self.STATE_KEYS}
        st = HybState()
        for k in self.STATE_KEYS:
            setattr(st, k, C.cast(self._tabs[k], _lib.PP))
        st.n_seq, st.t_max = self.n_seq, self.t_max
        self.state = st

    def ensure_sequences(self, n_seq):
        """Grow the caches and states to `n_seq` cache sequences; the existing ones keep their contents."""
        if n_seq <= self.n_seq:
            return
        need = n_seq * self.state_bytes_per_sequence()
        free, _ = torch.cuda.mem_get_info(self.device)
        if need > free:
            raise MemoryError(f"{n_seq} cache sequences at t_max = {self.t_max} need {need / 2**30:.1f} GiB, {free / 2**30:.1f} GiB free")
        new = self._alloc_state(n_seq)
        for old_run, new_run in zip(self.state_t, new):
            for k, t in old_run.items():
                if t is not None:
                    new_run[k][:self.n_seq].copy_(t)
        self.state_t, self.n_seq = new, n_seq
        self._bind_state()

    def release_sequences(self, n_keep):
        """Shrink back to the first `n_keep` cache sequences."""
        if n_keep >= self.n_seq:
            return
        self.state_t = [{k: (None if t is None else t[:n_keep].clone()) for k, t in run.items()} for run in self.state_t]
        self.n_seq = n_keep
        self._bind_state()

    # ---- construction ---------------------------------------------------------------------------------------------------------
    @classmethod
    def from_pretrained(cls, path, device="cuda", **kw):
        """A directory with config.json and *.safetensors (bf16 tensors under the checkpoint's names)."""
        from .infer import load_safetensors_dir
        cfg = ZuzenexConfig.from_pretrained(path)
        if not glob.glob(os.path.join(path, "*.safetensors")):
            raise FileNotFoundError(f"{path}: no *.safetensors")
        sd = {k: v.to(device, torch.bfloat16) for k, v in load_safetensors_dir(path).items() if v.is_floating_point()}
        return cls(cfg, sd, **kw)

    @classmethod
    def synthetic(cls, cfg, device="cuda", seed=0, **kw):
        """Random weights of the architecture (synth.py's rule by tensor name)."""
        from .synth import synth_tensor
        sd = {}
        for k, shp in zuzenex_param_shapes(cfg).items():
            if k == "embed":
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=1.0)
            elif k.endswith("sink"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=1.0)
            elif k.endswith("correction"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=0.02)
            elif "norm" in k:
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=1.0, std=0.05)
            else:
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=shp[-1] ** -0.5)
        return cls(cfg, sd, **kw)

    # ---- stepping -------------------------------------------------------------------------------------------------------------
    def _workspace_bytes(self, rows, max_len):
        return lib().mn_hyb_workspace_bytes(C.byref(self.struct), rows)

    def max_rows(self):
        """Rows of one pass: the (row, expert) pairs of a pass are at most 65535."""
        top = max([int(ly["mlp"]["router"]["top"]) for ly in self.cfg.layers if ly.get("mlp") and ly["mlp"]["kind"] == "moe"] or [1])
        return max(1, min(super().max_rows(), 65535 // top))

    def step(self, x, row_seq, row_slot, row_back, row_len=None, blk_tab=None, max_len=None, out=None, trace=None, ws=None, distinct=False,
             chunk_tab=None):
        """One pass of the stack over M rows.  x fp32 [M, width] (input embeddings); int32 device arrays per row (row r is position
        row_slot[r] of cache sequence row_seq[r], preceded in this pass by row_back[r] rows of its sequence); blk_tab int32 [n_blk, 2]
        cuts the rows into runs of <= block_rows consecutive rows of one sequence (not read when distinct) and chunk_tab int32
        [n_chunks, 2] into chunks of <= chunk_rows (optional: without it the recurrences walk their rows one by one); row_len is the
        other decoder's table and is not read here; max_len (host int) >= every position + 1 (default: the cache's length).  Appends
        the rows' keys and values and advances the recurrent states.  trace: optional fp32 [runs, M, width] that receives the
        residual stream after every layer run.  distinct: every row is alone in its sequence (a decode step).  Returns the final
        norm's output [M, width] fp32."""
        M = x.shape[0]
        assert x.dtype == torch.float32 and x.is_cuda and x.stride(1) == 1 and x.shape[1] == self.cfg.width and 1 <= M <= self.max_rows()
        for t in (row_seq, row_slot, row_back):
            assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous() and t.numel() >= M
        max_len = self.t_max if max_len is None else int(max_len)
        assert 1 <= max_len <= self.t_max, f"{max_len} tokens exceed the cache (t_max = {self.t_max})"
        if not distinct:
            assert blk_tab is not None and blk_tab.dtype == torch.int32 and blk_tab.is_cuda and blk_tab.is_contiguous() and blk_tab.shape[1] == 2
        if chunk_tab is not None:
            assert chunk_tab.dtype == torch.int32 and chunk_tab.is_cuda and chunk_tab.is_contiguous() and chunk_tab.shape[1] == 2
        if out is None:
            out = torch.empty(M, self.cfg.width, dtype=torch.float32, device=self.device)
        if trace is not None:
            assert trace.dtype == torch.float32 and trace.is_contiguous() and tuple(trace.shape) == (self.n_trace, M, self.cfg.width)
        if ws is None:
            ws = self._workspace(M, max_len)
        use_chunks = chunk_tab is not None and not distinct
        check(lib().mn_hyb_step(C.byref(self.struct), C.byref(self.state), ptr(x), x.stride(0), M, ptr(row_seq), ptr(row_slot), ptr(row_back),
                                None if distinct else ptr(blk_tab), M if distinct else blk_tab.shape[0],
                                ptr(chunk_tab) if use_chunks else None, chunk_tab.shape[0] if use_chunks else 0, max_len,
                                1 if distinct else 0, ptr(out), ptr(trace), ptr(ws), ws.numel(), current_stream()), "mn_hyb_step")
        return out


class ZuzenexForCausalLM(SeqCausalLM):
    """`SeqCausalLM` over a `ZuzenexDecoder`."""

    @classmethod
    def from_pretrained(cls, path, device="cuda", t_max=2048, arith="bf16", eos_token_id=None):
        return cls(ZuzenexDecoder.from_pretrained(path, device=device, t_max=t_max, arith=arith), eos_token_id)
