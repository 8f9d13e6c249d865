"""Daberax: a decoder-only language model of post-norm layers, served by libmingnative's post-norm step function (mingnative.h
section 12: mn_pn_step).

Per layer, with x the fp32 residual stream of a token and rms(y) = y / sqrt(mean(y^2) + eps):
    x += w1 rms(mixer(x))                           the sublayers read x itself; the norm sits on their RESULT
    x += w2 rms(W_down (gelu(W_gate x) * W_up x))   gelu in its tanh form (a layer may have no feed-forward)
    x += ws rms(P (gelu(G x) * e))                  e = the layer's slice of a second embedding row of the token (`token_side`)
    mixer "attention":        q, k, v = W x + b; RMS norm over the WHOLE q and k projections with weights; rotary pairs (2i, 2i + 1) on
                              the first rot.dims values of a head, frequencies optionally rescaled by wavelength; scores q . k * scale,
                              soft-capped by tanh; a sliding window; softmax; head h times sigmoid(W_g x)_h; W_o + b
    mixer "latent_attention": one latent c = w rms(W_dkv x)[: kv_rank] and one rotated key part per token are cached; per head the key is
                              [W_uk c ; rotated part], the value W_uv c; sliding window; W_o.  Served in absorbed form: the queries are
                              mapped into latent space, attend [c ; rotated part] with values c, and W_uv expands the result
    mixer "delta":            q, k (kv_heads) and v (heads) through a short causal filter and silu; q, k unit vectors; per head
                              S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q with beta = sigmoid(W_b x),
                              g = exp(-exp(A_log) softplus(W_a x + dt_bias)); per-head RMS norm times silu(W_g x); W_o
Then RMS with a weight and the vocabulary projection times `logit_scale`.

This module owns HBM residency, like the other decoders' modules:
  * weights bf16; everything a mixer projects from x is stacked at load into ONE matrix (attention [q ; k ; v ; g] with a stacked bias,
    latent [q ; dkv], delta [q ; k ; v ; b ; a ; g] with the three filters stacked), [gate ; up] of the feed-forward likewise; W_uk per
    head transposed; rotary frequencies computed once in double on the host; A_log and dt_bias as fp32 device vectors;
  * per layer: fp32 key / value arenas [n_seq, t_max, .] (attention), ONE fp32 arena [n_seq, t_max, kv_rank + rot_dim] (latent), or the
    filter state [n_seq, conv - 1, channels] and the fp32 recurrent state [n_seq, heads, dim, vdim] (delta); cache sequences are
    numbered as in the other decoders (`sequences.SequenceSlots`); a number that is given back is reused as it is: a row at position 0
    reads no state and positions bound every read;
  * per-row int32 bookkeeping on the device, so a lock-step decode loop never syncs with the host.
`arith`: "bf16" = matrix products of steps above 8 rows on the bf16 MFMA kernels (fp32 accumulate), everything else fp32;
"f32" = fp32 FMA everywhere.
"""
import ctypes as C
import glob
import os

import torch

from . import _lib
from ._lib import PnLayer, PnModel, PnState, check, current_stream, lib, ptr
from .configuration import DaberaxConfig, daberax_param_shapes
from .seq_lm import ARITH, SeqCausalLM, SeqDecoder

KIND = {"attention": 0, "latent_attention": 1, "delta": 2}
UNIT_EPS = 1e-6          # inside the root of the delta rule's unit norms: fixed by the design


def rotary_frequencies(rot, device):
    """fp32 device vector [dims / 2] of a mixer's `rot` dict(base, dims, optional scaling)."""
    dims = int(rot["dims"])
    sc = rot.get("scaling") or {}
    host = (C.c_float * max(1, dims // 2))()
    check(lib().mn_rotary_frequencies_scaled_host(dims, float(rot["base"]), float(sc.get("factor", 0.0)), float(sc.get("low", 0.0)),
                                                  float(sc.get("high", 0.0)), float(sc.get("original", 0.0)), host),
          "mn_rotary_frequencies_scaled_host")
    return torch.tensor(list(host), dtype=torch.float32, device=device)


class DaberaxDecoder(SeqDecoder):
    """Weights + per-layer caches and states + the C-ABI tables of the stack."""

    def __init__(self, cfg: DaberaxConfig, sd, t_max=2048, n_seq=1, arith="bf16"):
        """sd: {checkpoint tensor name: bf16 CUDA tensor}."""
        assert arith in ARITH, f"arith={arith!r}: 'bf16' or 'f32'"
        self.cfg, self.arith = cfg, arith
        missing = [k for k, shp in daberax_param_shapes(cfg).items() if k not in sd or tuple(sd[k].shape) != tuple(shp)]
        if missing:
            raise ValueError(f"checkpoint does not fit the configuration: missing or mis-shaped tensors {missing[:8]}")
        dev = sd["embed"].device
        self.device = dev
        self.embed_w, self.head_w = sd["embed"].contiguous(), sd["head"].contiguous()
        self.t_max, self.n_seq = int(t_max), int(n_seq)
        W, side = cfg.width, cfg.side_dim
        self.needs_tokens = side > 0
        self._keep = []                                  # packed tensors the C tables point to
        bf = dict(dtype=torch.bfloat16, device=dev)
        side_table = sd["side.embed"].contiguous() if side else None
        self._keep.append(side_table)
        layers = (PnLayer * len(cfg.layers))()
        self.dims = []                                   # per layer: the shapes of its caches and states
        for i, ly in enumerate(cfg.layers):
            m, mlp, p, L, t = ly["mixer"], ly.get("mlp"), f"l{i}.", layers[i], ly["type"]
            H, d, e = int(m["heads"]), int(m["dim"]), int(m["vdim"])
            L.kind, L.heads, L.dim, L.vdim = KIND[t], H, d, e
            L.norm1 = self._p(sd[p + "norm1"])
            bias = None
            if t == "attention":
                G = int(m["kv_heads"])
                L.kv_heads, L.scale, L.softcap, L.has_gate = G, float(m["scale"]), float(m.get("softcap") or 0.0), 1
                stack = [sd[p + "mix.q"], sd[p + "mix.k"], sd[p + "mix.v"], sd[p + "mix.g"]]
                bias = [sd[p + "mix.q.b"], sd[p + "mix.k.b"], sd[p + "mix.v.b"], torch.zeros(H, **bf)]
                L.q_norm, L.k_norm = self._p(sd[p + "mix.q.norm"]), self._p(sd[p + "mix.k.norm"])
                L.b_o = self._p(sd[p + "mix.o.b"])
                self.dims.append(dict(k=(G * d,), v=(G * e,)))
            elif t == "latent_attention":
                r, R = int(m["rot_dim"]), int(m["kv_rank"])
                L.kv_heads, L.rot, L.kv_rank, L.scale, L.softcap = 1, r, R, float(m["scale"]), float(m.get("softcap") or 0.0)
                stack = [sd[p + "mix.q"], sd[p + "mix.dkv"]]
                L.k_norm = self._p(sd[p + "mix.dkv.norm"])
                L.w_ukT = self._p(sd[p + "mix.uk"].reshape(H, d, R).transpose(1, 2))
                L.w_uv = self._p(sd[p + "mix.uv"])
                self.dims.append(dict(k=(int(lib().mn_pn_latent_ld(R, r)),)))
            else:
                G, taps = int(m["kv_heads"]), int(m["conv"])
                L.kv_heads, L.conv, L.unit_eps = G, taps, UNIT_EPS
                stack = [sd[p + "mix.q"], sd[p + "mix.k"], sd[p + "mix.v"], sd[p + "mix.b"], sd[p + "mix.a"], sd[p + "mix.g"]]
                L.w_conv = self._p(torch.cat([sd[p + "mix.q.conv"], sd[p + "mix.k.conv"], sd[p + "mix.v.conv"]], 0))
                L.a_log, L.dt_bias = self._f(sd[p + "mix.A_log"].float()), self._f(sd[p + "mix.dt_bias"].float())
                L.mix_norm = self._p(sd[p + "mix.norm"])
                self.dims.append(dict(conv=(taps - 1, 2 * G * d + H * e) if taps > 1 else None, lin=(H, d, e)))
            if t != "delta":
                rot = m.get("rot")
                if rot and int(rot["dims"]) > 0:
                    L.rot_dims, L.rot_interleaved = int(rot["dims"]), 1
                    L.rot_freq = self._f(rotary_frequencies(rot, dev))
                L.window = int((m.get("mask") or {}).get("size") or 0)
            rows = sum(x.shape[0] for x in stack)
            pad = -rows % 8                                              # zero rows: the stack's row count a multiple of 8
            L.w_in = self._p(torch.cat(stack + [torch.zeros(pad, W, **bf)], 0))
            if bias is not None:
                L.b_in = self._p(torch.cat(bias + [torch.zeros(pad, **bf)], 0))
            L.w_o = self._p(sd[p + "mix.o"])
            if mlp is not None:
                L.ff = int(mlp["ff"])
                L.norm2 = self._p(sd[p + "norm2"])
                L.w_gate_up = self._p(torch.cat([sd[p + "mlp.gate"], sd[p + "mlp.up"]], 0))
                L.w_down = self._p(sd[p + "mlp.down"])
            if side:
                L.side = side
                L.side_norm = self._p(sd[p + "side.norm"])
                L.w_side_gate = self._p(torch.cat([sd[p + "side.gate"], torch.zeros(-side % 8, W, **bf)], 0))
                L.w_side_proj = self._p(sd[p + "side.proj"])
                L.side_table = side_table.data_ptr() + 2 * i * side
        self._layers = layers
        self.n_trace = len(cfg.layers)
        s = PnModel()
        s.width, s.n_layers, s.arith, s.eps = W, len(cfg.layers), ARITH[arith], cfg.eps
        s.side_ld = side * len(cfg.layers)
        s.layers = C.cast(layers, C.POINTER(PnLayer))
        s.final_w = self._p(sd["final.norm"])
        self.struct = s
        self.state_t = self._alloc_state(self.n_seq)
        self._bind_state()
        self.block_rows = int(lib().mn_window_attn_block_rows())
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
    STATE_KEYS = ("k", "v", "conv", "lin")
    PER_TOKEN = ("k", "v")                              # arenas with one row per cached token

    def _state_shapes(self, n_seq):
        """Per layer: {name: shape or None}."""
        out = []
        for d in self.dims:
            out.append({k: (None if d.get(k) is None else ((n_seq, self.t_max) if k in self.PER_TOKEN else (n_seq,)) + tuple(d[k]))
                        for k in self.STATE_KEYS})
        return out

    def _alloc_state(self, n_seq):
        return [{k: (None if shp is None else torch.zeros(shp, dtype=torch.float32, device=self.device)) for k, shp in ly.items()}
                for ly in self._state_shapes(n_seq)]

    def state_bytes_per_sequence(self):
        return sum(4 * int(torch.Size(shp).numel()) for ly in self._state_shapes(1) for shp in ly.values() if shp is not None)

    def _bind_state(self):
        self._tabs = {k: _lib.ptr_array([ly[k] for ly in self.state_t]) for k in self.STATE_KEYS}
        st = PnState()
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
        for old_ly, new_ly in zip(self.state_t, new):
            for k, t in old_ly.items():
                if t is not None:
                    new_ly[k][:self.n_seq].copy_(t)
        self.state_t, self.n_seq = new, n_seq
        self._bind_state()

    def release_sequences(self, n_keep):
        """Shrink back to the first `n_keep` cache sequences."""
        if n_keep >= self.n_seq:
            return
        self.state_t = [{k: (None if t is None else t[:n_keep].clone()) for k, t in ly.items()} for ly in self.state_t]
        self.n_seq = n_keep
        self._bind_state()

    # ---- construction ---------------------------------------------------------------------------------------------------------
    @classmethod
    def from_pretrained(cls, path, device="cuda", **kw):
        """A directory with config.json and *.safetensors (bf16 tensors under the checkpoint's names)."""
        from .infer import load_safetensors_dir
        cfg = DaberaxConfig.from_pretrained(path)
        if not glob.glob(os.path.join(path, "*.safetensors")):
            raise FileNotFoundError(f"{path}: no *.safetensors")
        sd = {k: v.to(device, torch.bfloat16) for k, v in load_safetensors_dir(path).items() if v.is_floating_point()}
        return cls(cfg, sd, **kw)

    @classmethod
    def synthetic(cls, cfg, device="cuda", seed=0, **kw):
        """Random weights of the architecture (synth.py's rule by tensor name)."""
        from .synth import synth_tensor
        sd = {}
        for k, shp in daberax_param_shapes(cfg).items():
            if k in ("embed", "side.embed"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=1.0)
            elif k.endswith("A_log"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=-1.0, std=0.5)
            elif k.endswith("dt_bias"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=1.0)
            elif k.endswith(".b"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=0.05) if len(shp) == 1 else \
                    synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=shp[-1] ** -0.5)
            elif k.endswith(".conv"):
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=0.5)
            elif "norm" in k:
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=1.0, std=0.05)
            else:
                sd[k] = synth_tensor(k, shp, seed, device, torch.bfloat16, mean=0.0, std=shp[-1] ** -0.5)
        return cls(cfg, sd, **kw)

    # ---- stepping -------------------------------------------------------------------------------------------------------------
    def _workspace_bytes(self, rows, max_len):
        return lib().mn_pn_workspace_bytes(C.byref(self.struct), rows)

    def step(self, x, row_seq, row_slot, row_back, row_len=None, blk_tab=None, max_len=None, out=None, trace=None, ws=None, distinct=False,
             row_tok=None):
        """One pass of the stack over M rows.  x fp32 [M, width] (input embeddings); int32 device arrays per row (row r is token
        row_tok[r] at position row_slot[r] of cache sequence row_seq[r], preceded in this pass by row_back[r] rows of its sequence);
        blk_tab int32 [n_blk, 2] cuts the rows into runs of <= block_rows consecutive rows of one sequence (not read when distinct);
        row_len is the other decoders' table and is not read here; max_len (host int) >= every position + 1 (default: the cache's
        length).  Appends the rows' keys, values and latents and advances the filter and recurrent states.  trace: optional fp32
        [layers, M, width] that receives the residual stream after every layer.  distinct: every row is alone in its sequence (a decode
        step).  Returns the final norm's output [M, width] fp32."""
        M = x.shape[0]
        assert x.dtype == torch.float32 and x.is_cuda and x.stride(1) == 1 and x.shape[1] == self.cfg.width and 1 <= M <= self.max_rows()
        for t in (row_seq, row_slot, row_back):
            assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous() and t.numel() >= M
        if self.needs_tokens:
            assert row_tok is not None and row_tok.dtype == torch.int32 and row_tok.is_cuda and row_tok.is_contiguous() and row_tok.numel() >= M
        max_len = self.t_max if max_len is None else int(max_len)
        assert 1 <= max_len <= self.t_max, f"{max_len} tokens exceed the cache (t_max = {self.t_max})"
        if not distinct:
            assert blk_tab is not None and blk_tab.dtype == torch.int32 and blk_tab.is_cuda and blk_tab.is_contiguous() and blk_tab.shape[1] == 2
        if out is None:
            out = torch.empty(M, self.cfg.width, dtype=torch.float32, device=self.device)
        if trace is not None:
            assert trace.dtype == torch.float32 and trace.is_contiguous() and tuple(trace.shape) == (self.n_trace, M, self.cfg.width)
        if ws is None:
            ws = self._workspace(M, max_len)
        check(lib().mn_pn_step(C.byref(self.struct), C.byref(self.state), ptr(x), x.stride(0), M, ptr(row_tok), ptr(row_seq), ptr(row_slot),
                               ptr(row_back), None if distinct else ptr(blk_tab), M if distinct else blk_tab.shape[0], max_len,
                               1 if distinct else 0, ptr(out), ptr(trace), ptr(ws), ws.numel(), current_stream()), "mn_pn_step")
        return out

    # ---- vocabulary -----------------------------------------------------------------------------------------------------------
    def logits(self, hidden):
        """Vocabulary projection times `logit_scale` -> fp32 [M, vocab]."""
        out = super().logits(hidden)
        if self.cfg.logit_scale != 1.0:
            out.mul_(self.cfg.logit_scale)
        return out

    def greedy(self, hidden):
        """A positive scale leaves the arg-max where it is; any other goes through the scaled logits."""
        return super().greedy(hidden) if self.cfg.logit_scale > 0 else self.logits(hidden).argmax(-1)


class DaberaxForCausalLM(SeqCausalLM):
    """`SeqCausalLM` over a `DaberaxDecoder`."""

    @classmethod
    def from_pretrained(cls, path, device="cuda", t_max=2048, arith="bf16", eos_token_id=None):
        return cls(DaberaxDecoder.from_pretrained(path, device=device, t_max=t_max, arith=arith), eos_token_id)
