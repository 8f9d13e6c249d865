"""Configuration classes, field-compatible with the reference's.

  MingTokConfig        <- mingtok/modeling_mingtok.py:56-89 + config/config_mingtok.json
  BailingMoeConfig     <- mingunivision/configuration_bailing_moe.py:6-84
  MingUniVisionConfig  <- mingunivision/configuration_bailingmm.py:20-31
                          (+ `vishead_diffloss_config`, asserted at modeling_bailingmm.py:118)

  SakinexConfig        <- a decoder-only language model of parallel-mixer layers (windowed attention beside a minGRU, mixture-of-
                          experts feed-forward; no reference counterpart)
  DaberaxConfig        <- a decoder-only language model of post-norm layers (attention, latent attention or the gated delta rule per
                          layer, a per-layer token input; no reference counterpart)
  PizitarConfig        <- a decoder-only language model of latent-attention layers (no reference counterpart): config.json keys
                          `architecture`, `width`, `vocab`, `layers`, `canon.taps`, `norm.eps`, `logit_softcap`

`config_from_pretrained(dir)` picks the class by what config.json says (MODEL_REGISTRY).

Plain Python (no transformers dependency): `from_dict` / `to_dict` /
`from_json_file` / `from_pretrained(dir)` read the same JSON the reference's HF
configs serialise to; unknown keys are kept as attributes like PretrainedConfig does.
"""
import copy
import json
import os


class _Config:
    model_type = ""

    def __init__(self, **kwargs):
        for k, v in kwargs.items():
            setattr(self, k, v)

    @classmethod
    def from_dict(cls, d):
        d = dict(d)
        d.pop("model_type", None)
        return cls(**d)

    @classmethod
    def from_json_file(cls, path):
        with open(path) as f:
            return cls.from_dict(json.load(f))

    @classmethod
    def from_pretrained(cls, path):
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        return cls.from_json_file(path)

    def to_dict(self):
        out = {}
        for k, v in self.__dict__.items():
            out[k] = v.to_dict() if isinstance(v, _Config) else copy.deepcopy(v)
        out["model_type"] = self.model_type
        return out

    def to_json_string(self):
        return json.dumps(self.to_dict(), indent=2, sort_keys=True)

    def __repr__(self):
        return f"{type(self).__name__} {self.to_json_string()}"


class MingTokConfig(_Config):
    """MingTok-Vision hyper-parameters (mingtok/config/config_mingtok.json)."""
    model_type = "mingtok"

    def __init__(self, low_level_encoder=None, semantic_decoder=None, pixel_decoder=None,
                 scaling_factor=8.09449291, mean=1.46817409, model_dtype="bf16",
                 pretrained_checkpoint="", **kwargs):
        self.low_level_encoder = dict(low_level_encoder or dict(
            img_size=512, patch_size=32, depth=12, embed_dim=768, ffn_layer="swiglufused", out_dim=32))
        self.semantic_decoder = dict(semantic_decoder or dict(
            in_dim=32, patch_size=32, embed_dim=1024, decoder_depth=24, ffn_layer="swiglufused"))
        self.pixel_decoder = dict(pixel_decoder or dict(
            patch_size=16, decoder_depth=24, norm_pix_loss=True, embed_dim=1024, loss_type="L1-plain"))
        self.scaling_factor = scaling_factor
        self.mean = mean
        self.model_dtype = model_dtype
        self.pretrained_checkpoint = pretrained_checkpoint
        super().__init__(**kwargs)


class BailingMoeConfig(_Config):
    """Defaults follow configuration_bailing_moe.py:9-47."""
    model_type = "bailing_moe"

    def __init__(self, vocab_size=30592, hidden_size=1024, intermediate_size=None, num_hidden_layers=24,
                 num_attention_heads=16, num_key_value_heads=0, hidden_act="silu", use_qkv_bias=False,
                 use_bias=True, rms_norm_eps=1e-05, norm_head=False, tie_word_embeddings=False,
                 embedding_dropout=0.1, attention_dropout=0.1, output_dropout=0.1, initializer_range=0.02,
                 max_position_embeddings=16384, rope_theta=10000.0, use_cache=True, use_sliding_window=False,
                 sliding_window=4096, max_window_layers=28, rope_scaling=None, pad_token_id=126081,
                 num_experts=16, num_shared_experts=0, num_experts_per_tok=2, num_image_tokens_for_gen=256,
                 norm_topk_prob=True, moe_intermediate_size=None, first_k_dense_replace=0, head_dim=None,
                 output_router_logits=False, multi_gate=False, image_patch_token=126346,
                 image_start_token=126347, eos_token_id=126081, **kwargs):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.num_hidden_layers = num_hidden_layers
        self.num_attention_heads = num_attention_heads
        self.num_key_value_heads = num_key_value_heads
        self.hidden_act = hidden_act
        self.use_qkv_bias = use_qkv_bias
        self.use_bias = use_bias
        self.norm_head = norm_head
        self.rms_norm_eps = rms_norm_eps
        self.tie_word_embeddings = tie_word_embeddings
        self.embedding_dropout = embedding_dropout
        self.attention_dropout = attention_dropout
        self.output_dropout = output_dropout
        self.initializer_range = initializer_range
        self.max_position_embeddings = max_position_embeddings
        self.rope_theta = rope_theta
        self.use_cache = use_cache
        self.use_sliding_window = use_sliding_window
        self.sliding_window = sliding_window
        self.max_window_layers = max_window_layers
        self.head_dim = head_dim or self.hidden_size // self.num_attention_heads
        self.rope_scaling = rope_scaling
        self.pad_token_id = pad_token_id
        self.eos_token_id = eos_token_id
        self.num_experts = num_experts
        self.num_shared_experts = num_shared_experts
        self.num_experts_per_tok = num_experts_per_tok
        self.num_image_tokens_for_gen = num_image_tokens_for_gen
        self.norm_topk_prob = norm_topk_prob
        self.moe_intermediate_size = moe_intermediate_size
        self.first_k_dense_replace = first_k_dense_replace
        self.output_router_logits = output_router_logits
        self.multi_gate = multi_gate
        self.image_patch_token = image_patch_token
        self.image_start_token = image_start_token
        super().__init__(**kwargs)

    @classmethod
    def ming_univision_16b_a3b(cls):
        """The `llm_config` block of mingunivision/config.json:27-119 (Ling-lite 16.8B-A2.75B);
        rope_scaling forced to None: the hot path uses the Legacy rotary."""
        return cls(vocab_size=126464, hidden_size=2048, intermediate_size=5632, num_hidden_layers=28,
                   num_attention_heads=16, num_key_value_heads=4, head_dim=128, use_qkv_bias=False,
                   use_bias=False, rms_norm_eps=1e-5, rope_theta=600000, max_position_embeddings=32768,
                   num_experts=64, num_shared_experts=2, num_experts_per_tok=6, moe_intermediate_size=1408,
                   norm_topk_prob=True, multi_gate=True, first_k_dense_replace=0, initializer_range=0.006,
                   embedding_dropout=0.0, attention_dropout=0.0, output_dropout=0.0, rope_scaling=None)


DEFAULT_VISHEAD_DIFFLOSS = dict(  # defaults of setup_vishead_diffloss, modeling_bailing_moe.py:1559-1567
    diffloss_w=3072, diffloss_d=12, num_sampling_steps="16", gen_method="flow_matching_swiglu-4",
    vis_head_arch="linear2-norm")


class MingUniVisionConfig(_Config):
    model_type = "mingunivision"

    def __init__(self, mlp_depth=1, llm_config=None, vishead_diffloss_config=None, mingtok_config=None, **kwargs):
        self.llm_config = BailingMoeConfig.from_dict(llm_config) if isinstance(llm_config, dict) else llm_config
        self.mlp_depth = mlp_depth
        self.vishead_diffloss_config = dict(vishead_diffloss_config) if vishead_diffloss_config is not None else None
        # The reference hard-codes MingTok.from_pretrained("./models/MingTok-Vision")
        # (modeling_bailingmm.py:102); we let the tokenizer config ride along.
        self.mingtok_config = (MingTokConfig.from_dict(mingtok_config) if isinstance(mingtok_config, dict)
                               else mingtok_config)
        super().__init__(**kwargs)

    @classmethod
    def ming_univision_16b_a3b(cls):
        return cls(mlp_depth=2, llm_config=BailingMoeConfig.ming_univision_16b_a3b(),
                   vishead_diffloss_config=dict(DEFAULT_VISHEAD_DIFFLOSS), mingtok_config=MingTokConfig())


def swiglu_hidden(dim, mlp_ratio=4.0):
    """SwiGLUFFNFused hidden size (layers/swiglu_ffn.py:54-66; diff_loss_rf_swiglu.py:54-66)."""
    return (int(int(dim * mlp_ratio) * 2 / 3) + 7) // 8 * 8


# --------------------------------------------------------------------------
# parameter name -> shape tables (reference state-dict names)
# --------------------------------------------------------------------------
def _vit_block_shapes(prefix, D, ffn):
    s = {
        f"{prefix}.norm1.weight": (D,), f"{prefix}.norm1.bias": (D,),
        f"{prefix}.attn.qkv.weight": (3 * D, D), f"{prefix}.attn.qkv.bias": (3 * D,),
        f"{prefix}.attn.proj.weight": (D, D), f"{prefix}.attn.proj.bias": (D,),
        f"{prefix}.norm2.weight": (D,), f"{prefix}.norm2.bias": (D,),
    }
    if ffn == "swiglufused":
        h = swiglu_hidden(D)
        s.update({f"{prefix}.mlp.w12.weight": (2 * h, D), f"{prefix}.mlp.w12.bias": (2 * h,),
                  f"{prefix}.mlp.w3.weight": (D, h), f"{prefix}.mlp.w3.bias": (D,)})
    else:
        s.update({f"{prefix}.mlp.fc1.weight": (4 * D, D), f"{prefix}.mlp.fc1.bias": (4 * D,),
                  f"{prefix}.mlp.fc2.weight": (D, 4 * D), f"{prefix}.mlp.fc2.bias": (D,)})
    return s


def mingtok_param_shapes(cfg: MingTokConfig):
    enc, sem, pix = cfg.low_level_encoder, cfg.semantic_decoder, cfg.pixel_decoder
    s = {}
    De, P = enc.get("embed_dim", 1024), enc.get("patch_size", 16)
    n_pos = (enc.get("img_size", 224) // P) ** 2 + 1
    s["low_level_encoder.cls_token"] = (1, 1, De)
    s["low_level_encoder.pos_embed"] = (1, n_pos, De)
    s["low_level_encoder.patch_embed.proj.weight"] = (De, 3, P, P)
    s["low_level_encoder.patch_embed.proj.bias"] = (De,)
    for i in range(enc.get("depth", 24)):
        s.update(_vit_block_shapes(f"low_level_encoder.blocks.0.{i}", De, enc.get("ffn_layer", "mlp")))
    s["low_level_encoder.out_norm.weight"] = (De,)
    s["low_level_encoder.out_norm.bias"] = (De,)
    s["low_level_encoder.out_proj.weight"] = (enc["out_dim"], De)
    s["low_level_encoder.out_proj.bias"] = (enc["out_dim"],)
    Ds = sem.get("embed_dim", 1024)
    s["semantic_decoder.in_proj.weight"] = (Ds, sem["in_dim"])
    s["semantic_decoder.in_proj.bias"] = (Ds,)
    for i in range(sem.get("decoder_depth", 1)):
        s.update(_vit_block_shapes(f"semantic_decoder.blocks.0.{i}", Ds, sem.get("ffn_layer", "mlp")))
    s["semantic_decoder.norm.weight"] = (Ds,)
    s["semantic_decoder.norm.bias"] = (Ds,)
    Dp, Pp = pix.get("embed_dim", 1024), pix.get("patch_size", 16)
    for i in range(pix.get("decoder_depth", 1)):
        s.update(_vit_block_shapes(f"pixel_decoder.blocks.0.{i}", Dp, "mlp"))
    s["pixel_decoder.norm.weight"] = (Dp,)
    s["pixel_decoder.norm.bias"] = (Dp,)
    s["pixel_decoder.head.weight"] = (Pp * Pp * 3, Dp)
    s["pixel_decoder.head.bias"] = (Pp * Pp * 3,)
    ratio = sem.get("patch_size", 16) // Pp
    s["sem_to_pix.weight"] = (Dp * ratio * ratio, Ds)
    s["sem_to_pix.bias"] = (Dp * ratio * ratio,)
    return s


def rf_param_shapes(w, depth, z_channels, target=32, mlp_mult=4, prefix="diffloss."):
    h = swiglu_hidden(w, mlp_mult)
    p = prefix + "net."
    s = {
        p + "time_embed.mlp.0.weight": (w, 256), p + "time_embed.mlp.0.bias": (w,),
        p + "time_embed.mlp.2.weight": (w, w), p + "time_embed.mlp.2.bias": (w,),
        p + "cond_embed.weight": (w, z_channels), p + "cond_embed.bias": (w,),
        p + "input_proj.weight": (w, target), p + "input_proj.bias": (w,),
    }
    for i in range(depth):
        b = f"{p}res_blocks.{i}."
        s.update({b + "in_ln.weight": (w,), b + "in_ln.bias": (w,),
                  b + "mlp.w12.weight": (2 * h, w), b + "mlp.w12.bias": (2 * h,),
                  b + "mlp.w3.weight": (w, h), b + "mlp.w3.bias": (w,),
                  b + "adaLN_modulation.1.weight": (3 * w, w), b + "adaLN_modulation.1.bias": (3 * w,)})
    f = p + "final_layer."
    s.update({f + "linear.weight": (target, w), f + "linear.bias": (target,),
              f + "adaLN_modulation.1.weight": (2 * w, w), f + "adaLN_modulation.1.bias": (2 * w,)})
    return s


def llm_layer_param_shapes(cfg: BailingMoeConfig, li, prefix="model.layers."):
    H, hd = cfg.hidden_size, cfg.head_dim
    nq, nkv, I = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.moe_intermediate_size
    p = f"{prefix}{li}."
    s = {p + "input_layernorm.weight": (H,), p + "post_attention_layernorm.weight": (H,),
         p + "attention.query_key_value.weight": ((nq + 2 * nkv) * hd, H),
         p + "attention.dense.weight": (H, nq * hd)}
    if cfg.use_qkv_bias:
        s[p + "attention.query_key_value.bias"] = ((nq + 2 * nkv) * hd,)
    if cfg.use_bias:
        s[p + "attention.dense.bias"] = (H,)
    gates = ["gate"] + (["image_gate", "audio_gate"] if cfg.multi_gate else [])
    for g in gates:
        s[p + f"mlp.{g}.weight"] = (cfg.num_experts, H)
    for e in range(cfg.num_experts):
        s[p + f"mlp.experts.{e}.gate_proj.weight"] = (I, H)
        s[p + f"mlp.experts.{e}.up_proj.weight"] = (I, H)
        s[p + f"mlp.experts.{e}.down_proj.weight"] = (H, I)
    if cfg.num_shared_experts:
        Is = I * cfg.num_shared_experts
        s[p + "mlp.shared_experts.gate_proj.weight"] = (Is, H)
        s[p + "mlp.shared_experts.up_proj.weight"] = (Is, H)
        s[p + "mlp.shared_experts.down_proj.weight"] = (H, Is)
    return s


def llm_param_shapes(cfg: BailingMoeConfig, vishead_diffloss_config=None, latent_dim=32):
    """Names of BailingMoeForCausalLM (+ vis_head / diffloss when configured)."""
    s = {"model.word_embeddings.weight": (cfg.vocab_size, cfg.hidden_size)}
    for li in range(cfg.num_hidden_layers):
        s.update(llm_layer_param_shapes(cfg, li))
    s["model.norm.weight"] = (cfg.hidden_size,)
    s["lm_head.weight"] = (cfg.vocab_size, cfg.hidden_size)
    if vishead_diffloss_config is not None:
        c = {**DEFAULT_VISHEAD_DIFFLOSS, **vishead_diffloss_config}
        w = c["diffloss_w"]
        s["vis_head.0.weight"] = (w, cfg.hidden_size)
        s["vis_head.0.bias"] = (w,)
        s["vis_head.1.weight"] = (w,)
        s["vis_head.1.bias"] = (w,)
        s.update(rf_param_shapes(w, c["diffloss_d"], w, latent_dim, int(c["gen_method"].split("-")[1])))
    return s


def linear_proj_param_shapes(feature_dim, hidden_size, mlp_depth, prefix="linear_proj."):
    s = {prefix + "0.weight": (hidden_size, feature_dim), prefix + "0.bias": (hidden_size,)}
    for i in range(1, mlp_depth):
        s[prefix + f"{2 * i}.weight"] = (hidden_size, hidden_size)
        s[prefix + f"{2 * i}.bias"] = (hidden_size,)
    return s


# ---- Pizitar ---------------------------------------------------------------------------------------------------------------
PIZITAR_MIXERS = ("latent_attention", "latent_attention_2")


class PizitarConfig(_Config):
    """A stack of latent-attention layers.  `layers` is a list of dicts(type, mixer, mlp):
    type  "latent_attention"   queries through an RMS-normed latent of `q_rank` rows; optional `kv_from`: j = attend layer j's cached
                               latents (this layer then has no kv projection of its own)
          "latent_attention_2" direct queries and a sigmoid gate on the concatenated heads
    mixer heads, dim (query / key size per head), vdim, kv_rank (size of the cached latent), scale (of the scores)
    mlp   None or dict(kind="dense", ff)
    Every size is read from here or from the tensors; nothing is assumed equal between layers."""
    model_type = "pizitar"

    def __init__(self, width=256, vocab=1024, layers=(), canon=None, norm=None, logit_softcap=None, architecture="Pizitar", **kwargs):
        self.architecture = architecture
        self.width, self.vocab = int(width), int(vocab)
        self.layers = [copy.deepcopy(dict(ly)) for ly in layers]
        self.canon = dict(canon or {"taps": 1})
        self.norm = dict(norm or {"eps": 1e-6})
        self.logit_softcap = logit_softcap
        super().__init__(**kwargs)
        self.validate()

    taps = property(lambda self: int(self.canon["taps"]))
    eps = property(lambda self: float(self.norm["eps"]))

    def validate(self):
        if self.taps < 1:
            raise ValueError("canon.taps must be >= 1")
        for i, ly in enumerate(self.layers):
            if ly.get("type") not in PIZITAR_MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {ly.get('type')!r} (known: {PIZITAR_MIXERS})")
            m = ly["mixer"]
            for k in ("heads", "dim", "vdim", "kv_rank", "scale"):
                if k not in m:
                    raise ValueError(f"layer {i}: mixer lacks {k!r}")
            if ly["type"] == "latent_attention" and "q_rank" not in m:
                raise ValueError(f"layer {i}: latent_attention needs q_rank")
            src = m.get("kv_from")
            if src is not None:
                if ly["type"] != "latent_attention":
                    raise ValueError(f"layer {i}: kv_from is a latent_attention option")
                if not (0 <= src < i) or self.layers[src]["mixer"].get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from = {src} must name an earlier layer that projects its own latent")
                if self.layers[src]["mixer"]["kv_rank"] != m["kv_rank"]:
                    raise ValueError(f"layer {i}: kv_rank differs from layer {src}'s, whose latents it attends")
            mlp = ly.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")


def pizitar_param_shapes(cfg: PizitarConfig):
    """{tensor name: shape} of a Pizitar checkpoint (`l<i>.` per layer; `.b` = the bias of the tensor it follows)."""
    W, V, taps = cfg.width, cfg.vocab, cfg.taps
    s = {"embed": (V, W)}
    for i, ly in enumerate(cfg.layers):
        p, m, mlp = f"l{i}.", ly["mixer"], ly.get("mlp")
        H, d, v, r = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if mlp is not None else ()):
            s[p + n], s[p + n + ".b"] = (W,), (W,)
        if ly["type"] == "latent_attention":
            s[p + "mix.dq"], s[p + "mix.dq.norm"], s[p + "mix.uq"] = (m["q_rank"], W), (m["q_rank"],), (H * d, m["q_rank"])
        else:
            s[p + "mix.q"], s[p + "mix.g"] = (H * d, W), (H * v, W)
        if m.get("kv_from") is None:
            s[p + "mix.dkv"], s[p + "mix.dkv.norm"] = (r, W), (r,)
        s[p + "mix.uk"], s[p + "mix.uv"], s[p + "mix.o"] = (H * d, r), (H * v, r), (W, H * v)
        if mlp is not None:
            s[p + "mlp.up"], s[p + "mlp.down"], s[p + "mlp.act"] = (mlp["ff"], W), (W, mlp["ff"]), (4,)
            s[p + "rg2"], s[p + "rg2.b"] = (W, W), (W,)
        s[p + "canon1"] = (W, taps)
        s[p + "rg1"], s[p + "rg1.b"] = (W, W), (W,)
    s["final.norm"], s["final.norm.b"], s["head"] = (W,), (W,), (V, W)
    return s


# ---- Sakinex ---------------------------------------------------------------------------------------------------------------
SAKINEX_MIXERS = ("parallel",)


class SakinexConfig(_Config):
    """A stack of parallel-mixer layers.  `layers` is a list of dicts(type, mixer, mlp):
    type  "parallel": a windowed attention (`mixer.left`) beside a minGRU (`mixer.right`), summed with `left_scale` / `right_scale`
    left  heads, kv_heads, dim (query / key size per head), vdim, scale (of the scores); optional conv (taps of the filter on the
          projected q / k / v channels), rot dict(base, dims, optional scaling dict(factor, original, fast, slow)), mask
          dict(size = window, optional pool = tokens per pooled block before the window); no mask: every earlier token
    right width
    mlp   None or dict(kind="moe", router dict(experts, top), expert dict(ff), optional shared dict(ff))
    canon dict(taps): the causal filter added to what every sublayer reads (absent: none); loop dict(start, stop, times): layers
    start .. stop - 1 run `times` times in a row with the same weights.  Every size is read from here or from the tensors; nothing
    is assumed equal between layers."""
    model_type = "sakinex"

    def __init__(self, width=256, vocab=1024, layers=(), canon=None, norm=None, loop=None, residual_mult=1.0, architecture="Sakinex",
                 **kwargs):
        self.architecture = architecture
        self.width, self.vocab = int(width), int(vocab)
        self.layers = [copy.deepcopy(dict(ly)) for ly in layers]
        self.canon = dict(canon) if canon else None
        self.norm = dict(norm or {"eps": 1e-6})
        self.loop = dict(loop) if loop else None
        self.residual_mult = float(residual_mult)
        super().__init__(**kwargs)
        self.validate()

    taps = property(lambda self: int(self.canon["taps"]) if self.canon else 0)
    eps = property(lambda self: float(self.norm["eps"]))

    def runs(self):
        """[(layer, add the embedding rows first)] in execution order."""
        n = len(self.layers)
        if not self.loop:
            return [(i, False) for i in range(n)]
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        out = [(i, False) for i in range(a)]
        for r in range(times):
            out += [(i, r > 0 and i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, n)]

    def validate(self):
        if self.canon and self.taps < 1:
            raise ValueError("canon.taps must be >= 1")
        if self.loop:
            a, b, times = (int(self.loop[k]) for k in ("start", "stop", "times"))
            if not (0 <= a <= b <= len(self.layers)) or times < 1:
                raise ValueError(f"loop {self.loop}: 0 <= start <= stop <= {len(self.layers)} layers and times >= 1")
        for i, ly in enumerate(self.layers):
            if ly.get("type") not in SAKINEX_MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {ly.get('type')!r} (known: {SAKINEX_MIXERS})")
            m = ly["mixer"]
            for k in ("left", "right", "left_scale", "right_scale"):
                if k not in m:
                    raise ValueError(f"layer {i}: mixer lacks {k!r}")
            L = m["left"]
            for k in ("heads", "kv_heads", "dim", "vdim", "scale"):
                if k not in L:
                    raise ValueError(f"layer {i}: mixer.left lacks {k!r}")
            if L["heads"] % L["kv_heads"]:
                raise ValueError(f"layer {i}: {L['heads']} query heads do not divide over {L['kv_heads']} key/value heads")
            rot = L.get("rot")
            if rot and (rot["dims"] % 2 or rot["dims"] > L["dim"]):
                raise ValueError(f"layer {i}: rot.dims = {rot['dims']} must be even and at most dim = {L['dim']}")
            mask = L.get("mask")
            if mask and (int(mask["size"]) < 1 or int(mask.get("pool") or 1) < 1):
                raise ValueError(f"layer {i}: mask {mask}: size >= 1, pool >= 1")
            if "width" not in m["right"]:
                raise ValueError(f"layer {i}: mixer.right lacks 'width'")
            mlp = ly.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                if not (1 <= int(mlp["router"]["top"]) <= int(mlp["router"]["experts"])):
                    raise ValueError(f"layer {i}: router {mlp['router']}: 1 <= top <= experts")


def sakinex_param_shapes(cfg: SakinexConfig):
    """{tensor name: shape} of a Sakinex checkpoint (`l<i>.` per layer; `.b` = the bias and `.conv` the filter of the tensor it follows)."""
    W, V, taps = cfg.width, cfg.vocab, cfg.taps
    s = {"embed": (V, W)}
    for i, ly in enumerate(cfg.layers):
        p, m, mlp = f"l{i}.", ly["mixer"], ly.get("mlp")
        L, wr = m["left"], int(m["right"]["width"])
        H, G, d, e = int(L["heads"]), int(L["kv_heads"]), int(L["dim"]), int(L["vdim"])
        s[p + "norm1"] = (W,)
        for n, rows in (("q", H * d), ("k", G * d), ("v", G * e)):
            s[p + "mix.left." + n] = (rows, W)
            if L.get("conv"):
                s[p + "mix.left." + n + ".conv"] = (rows, int(L["conv"]))
        s[p + "mix.left.o"] = (W, H * e)
        for n in ("z", "x"):
            s[p + "mix.right." + n], s[p + "mix.right." + n + ".b"] = (wr, W), (wr,)
        s[p + "mix.right.g"], s[p + "mix.right.o"] = (wr, W), (W, wr)
        if taps:
            s[p + "canon1"] = (W, taps)
        if mlp is not None:
            s[p + "norm2"] = (W,)
            E, ff = int(mlp["router"]["experts"]), int(mlp["expert"]["ff"])
            for j in range(E):
                s[f"{p}mlp.e{j}.gate"], s[f"{p}mlp.e{j}.up"], s[f"{p}mlp.e{j}.down"] = (ff, W), (ff, W), (W, ff)
            s[p + "mlp.router"], s[p + "mlp.router.b"] = (E, W), (E,)
            if mlp.get("shared"):
                fs = int(mlp["shared"]["ff"])
                s[p + "mlp.shared.gate"], s[p + "mlp.shared.up"], s[p + "mlp.shared.down"] = (fs, W), (fs, W), (W, fs)
                s[p + "mlp.shared.sg"] = (1, W)
            if taps:
                s[p + "canon2"] = (W, taps)
    s["final.norm"], s["head"] = (W,), (V, W)
    return s


# ---- Zuzenex ---------------------------------------------------------------------------------------------------------------
ZUZENEX_MIXERS = ("attention", "lightning")


class ZuzenexConfig(_Config):
    """A stack of layers that run their mixer and their feed-forward in parallel on one normed input.  `layers` is a list of
    dicts(type, mixer, mlp):
    type  "attention": causal softmax attention — mixer dict(heads, kv_heads, dim, vdim, scale, optional q_temp dict(coef, every)):
                       queries and keys RMS-normed per head with a weight, the query at position p multiplied by
                       1 + coef ln(floor((p + 1) / every) + 1), one learned sink per head in the softmax's denominator
          "lightning": decayed linear attention — mixer dict(heads, dim, vdim, decay = one factor per head)
    mlp   None, dict(kind="dense", ff) or dict(kind="moe", router dict(experts, top, optional identity = router outputs past the
          experts that pass the input through), expert dict(ff), optional shared dict(ff))
    loop  dict(start, stop, times): layers start .. stop - 1 run `times` times in a row with the same weights (every run owns its cache
    or state).  Every size is read from here or from the tensors; nothing is assumed equal between layers."""
    model_type = "zuzenex"

    def __init__(self, width=256, vocab=1024, layers=(), norm=None, loop=None, architecture="Zuzenex", **kwargs):
        self.architecture = architecture
        self.width, self.vocab = int(width), int(vocab)
        self.layers = [copy.deepcopy(dict(ly)) for ly in layers]
        self.norm = dict(norm or {"eps": 1e-6})
        self.loop = dict(loop) if loop else None
        super().__init__(**kwargs)
        self.validate()

    eps = property(lambda self: float(self.norm["eps"]))

    def runs(self):
        """The layer of every run, in execution order."""
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    def validate(self):
        if self.loop:
            a, b, times = (int(self.loop[k]) for k in ("start", "stop", "times"))
            if not (0 <= a <= b <= len(self.layers)) or times < 1:
                raise ValueError(f"loop {self.loop}: 0 <= start <= stop <= {len(self.layers)} layers and times >= 1")
        for i, ly in enumerate(self.layers):
            if ly.get("type") not in ZUZENEX_MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {ly.get('type')!r} (known: {ZUZENEX_MIXERS})")
            m = ly["mixer"]
            need = ("heads", "kv_heads", "dim", "vdim", "scale") if ly["type"] == "attention" else ("heads", "dim", "vdim", "decay")
            for k in need:
                if k not in m:
                    raise ValueError(f"layer {i}: mixer lacks {k!r}")
            if ly["type"] == "attention":
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ValueError(f"layer {i}: {m['heads']} query heads do not divide over {m['kv_heads']} key/value heads")
                qt = m.get("q_temp")
                if qt and int(qt["every"]) < 1:
                    raise ValueError(f"layer {i}: q_temp.every must be >= 1")
            elif len(m["decay"]) != int(m["heads"]):
                raise ValueError(f"layer {i}: {len(m['decay'])} decay factors for {m['heads']} heads")
            mlp = ly.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind") == "dense":
                if int(mlp["ff"]) < 1:
                    raise ValueError(f"layer {i}: dense feed-forward needs ff >= 1")
            elif mlp.get("kind") == "moe":
                r = mlp["router"]
                if int(r["experts"]) < 1 or not (1 <= int(r["top"]) <= int(r["experts"]) + int(r.get("identity") or 0)):
                    raise ValueError(f"layer {i}: router {r}: experts >= 1 and 1 <= top <= experts + identity")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")


def zuzenex_param_shapes(cfg: ZuzenexConfig):
    """{tensor name: shape} of a Zuzenex checkpoint (`l<i>.` per layer, `mix.` the mixer's and `mlp.` the feed-forward's tensors)."""
    W, V = cfg.width, cfg.vocab
    s = {"embed": (V, W)}
    for i, ly in enumerate(cfg.layers):
        p, m, mlp = f"l{i}.", ly["mixer"], ly.get("mlp")
        H, d, e = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        s[p + "norm1"] = (W,)
        if ly["type"] == "attention":
            G = int(m["kv_heads"])
            s[p + "mix.q"], s[p + "mix.k"], s[p + "mix.v"] = (H * d, W), (G * d, W), (G * e, W)
            s[p + "mix.q.norm"], s[p + "mix.k.norm"], s[p + "mix.sink"] = (d,), (d,), (H,)
        else:
            s[p + "mix.q"], s[p + "mix.k"], s[p + "mix.v"], s[p + "mix.g"] = (H * d, W), (H * d, W), (H * e, W), (H * e, W)
            s[p + "mix.norm"] = (H * e,)
        s[p + "mix.o"] = (W, H * e)
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            s[p + "mlp.up"], s[p + "mlp.down"] = (int(mlp["ff"]), W), (W, int(mlp["ff"]))
            continue
        r = mlp["router"]
        E, n_out, ff = int(r["experts"]), int(r["experts"]) + int(r.get("identity") or 0), int(mlp["expert"]["ff"])
        for j in range(E):
            s[f"{p}mlp.e{j}.up"], s[f"{p}mlp.e{j}.down"] = (ff, W), (W, ff)
        s[p + "mlp.router"], s[p + "mlp.correction"] = (n_out, W), (n_out,)
        if mlp.get("shared"):
            fs = int(mlp["shared"]["ff"])
            s[p + "mlp.shared.up"], s[p + "mlp.shared.down"] = (fs, W), (W, fs)
    s["final.norm"], s["head"] = (W,), (V, W)
    return s


# ---- Daberax ---------------------------------------------------------------------------------------------------------------
DABERAX_MIXERS = ("attention", "latent_attention", "delta")


class DaberaxConfig(_Config):
    """A stack of layers whose sublayers read the residual stream as it is and whose RESULTS are RMS-normed before they are added.
    `layers` is a list of dicts(type, mixer, mlp):
    type  "attention":        mixer dict(heads, kv_heads, dim, vdim, scale, optional rot dict(base, dims, optional scaling dict(factor,
                              low, high, original)), optional softcap, optional mask dict(size)): biases, RMS norm over the whole q and k
                              projections, interleaved rotary pairs, soft-capped scores, sliding window, a sigmoid gate per head
          "latent_attention": mixer dict(heads, dim, rot_dim, vdim, kv_rank, scale, rot dict(base, dims), optional softcap, optional
                              mask): one normed latent and one rotated key part per token, keys and values are linear maps of the latent
          "delta":            mixer dict(heads, kv_heads, dim, vdim, conv): the gated delta rule on filtered, unit-length q and k
    mlp   None or dict(kind="dense", ff)
    token_side dict(dim): every layer adds a normed projection of gelu(G x) * (its slice of a second embedding row of the token).
    Every size is read from here or from the tensors; nothing is assumed equal between layers."""
    model_type = "daberax"

    def __init__(self, width=256, vocab=1024, layers=(), norm=None, token_side=None, logit_scale=1.0, architecture="Daberax", **kwargs):
        self.architecture = architecture
        self.width, self.vocab = int(width), int(vocab)
        self.layers = [copy.deepcopy(dict(ly)) for ly in layers]
        self.norm = dict(norm or {"eps": 1e-6})
        self.token_side = dict(token_side) if token_side else None
        self.logit_scale = float(logit_scale)
        super().__init__(**kwargs)
        self.validate()

    eps = property(lambda self: float(self.norm["eps"]))
    side_dim = property(lambda self: int(self.token_side["dim"]) if self.token_side else 0)

    def validate(self):
        if self.token_side and int(self.token_side["dim"]) < 1:
            raise ValueError("token_side.dim must be >= 1")
        for i, ly in enumerate(self.layers):
            t = ly.get("type")
            if t not in DABERAX_MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {t!r} (known: {DABERAX_MIXERS})")
            m = ly["mixer"]
            need = {"attention": ("heads", "kv_heads", "dim", "vdim", "scale"),
                    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale"),
                    "delta": ("heads", "kv_heads", "dim", "vdim", "conv")}[t]
            for k in need:
                if k not in m:
                    raise ValueError(f"layer {i}: mixer lacks {k!r}")
            if t != "latent_attention" and int(m["heads"]) % int(m["kv_heads"]):
                raise ValueError(f"layer {i}: {m['heads']} heads do not divide over {m['kv_heads']} key heads")
            if t == "delta" and int(m["conv"]) < 1:
                raise ValueError(f"layer {i}: conv must be >= 1")
            rot = m.get("rot")
            if t == "latent_attention" and not rot and int(m["rot_dim"]) > 0:
                raise ValueError(f"layer {i}: latent attention with a rotated part needs rot")
            if rot and t != "delta":
                span = int(m["rot_dim"]) if t == "latent_attention" else int(m["dim"])
                if int(rot["dims"]) % 2 or not (0 <= int(rot["dims"]) <= span):
                    raise ValueError(f"layer {i}: rot.dims = {rot['dims']} must be even and at most {span}")
                sc = rot.get("scaling")
                if sc and not (0 < float(sc["low"]) < float(sc["high"]) and float(sc["factor"]) > 0 and float(sc["original"]) > 0):
                    raise ValueError(f"layer {i}: rot.scaling {sc}: 0 < low < high, factor > 0, original > 0")
            if m.get("mask") and int(m["mask"]["size"]) < 1:
                raise ValueError(f"layer {i}: mask.size must be >= 1")
            mlp = ly.get("mlp")
            if mlp is not None and (mlp.get("kind") != "dense" or int(mlp["ff"]) < 1):
                raise ValueError(f"layer {i}: feed-forward {mlp}: kind 'dense' with ff >= 1")


def daberax_param_shapes(cfg: DaberaxConfig):
    """{tensor name: shape} of a Daberax checkpoint (`l<i>.` per layer, `mix.` the mixer's, `mlp.` the feed-forward's and `side.` the
    token input's tensors)."""
    W, V, sd = cfg.width, cfg.vocab, cfg.side_dim
    s = {"embed": (V, W)}
    if sd:
        s["side.embed"] = (V, sd * len(cfg.layers))
    for i, ly in enumerate(cfg.layers):
        p, m, mlp, t = f"l{i}.", ly["mixer"], ly.get("mlp"), ly["type"]
        H, d, e = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        s[p + "norm1"] = (W,)
        if t == "attention":
            G = int(m["kv_heads"])
            s[p + "mix.q"], s[p + "mix.k"], s[p + "mix.v"] = (H * d, W), (G * d, W), (G * e, W)
            s[p + "mix.q.b"], s[p + "mix.k.b"], s[p + "mix.v.b"], s[p + "mix.o.b"] = (H * d,), (G * d,), (G * e,), (W,)
            s[p + "mix.q.norm"], s[p + "mix.k.norm"], s[p + "mix.g"] = (H * d,), (G * d,), (H, W)
        elif t == "latent_attention":
            r, R = int(m["rot_dim"]), int(m["kv_rank"])
            s[p + "mix.q"], s[p + "mix.dkv"], s[p + "mix.dkv.norm"] = (H * (d + r), W), (R + r, W), (R,)
            s[p + "mix.uk"], s[p + "mix.uv"] = (H * d, R), (H * e, R)
        else:
            G, taps = int(m["kv_heads"]), int(m["conv"])
            for n, rows in (("q", G * d), ("k", G * d), ("v", H * e)):
                s[p + "mix." + n], s[p + "mix." + n + ".conv"] = (rows, W), (rows, taps)
            s[p + "mix.b"], s[p + "mix.a"], s[p + "mix.A_log"], s[p + "mix.dt_bias"] = (H, W), (H, W), (H,), (H,)
            s[p + "mix.norm"], s[p + "mix.g"] = (e,), (H * e, W)
        s[p + "mix.o"] = (W, H * e)
        if mlp is not None:
            ff = int(mlp["ff"])
            s[p + "norm2"] = (W,)
            s[p + "mlp.gate"], s[p + "mlp.up"], s[p + "mlp.down"] = (ff, W), (ff, W), (W, ff)
        if sd:
            s[p + "side.gate"], s[p + "side.proj"], s[p + "side.norm"] = (sd, W), (W, sd), (W,)
    s["final.norm"], s["head"] = (W,), (V, W)
    return s


# ---- registry: which configuration class a config.json belongs to -------------------------------------------------------------
def _is_pizitar(d):
    return d.get("architecture") == "Pizitar" or d.get("model_type") == "pizitar"


def _is_sakinex(d):
    return d.get("architecture") == "Sakinex" or d.get("model_type") == "sakinex"


def _is_zuzenex(d):
    return d.get("architecture") == "Zuzenex" or d.get("model_type") == "zuzenex"


def _is_daberax(d):
    return d.get("architecture") == "Daberax" or d.get("model_type") == "daberax"


def _is_ming_univision(d):
    return "llm_config" in d or d.get("model_type") in ("bailingmm", "ming_univision")


MODEL_REGISTRY = [("pizitar", _is_pizitar, PizitarConfig), ("sakinex", _is_sakinex, SakinexConfig), ("zuzenex", _is_zuzenex, ZuzenexConfig),
                  ("daberax", _is_daberax, DaberaxConfig),
                  ("ming_univision", _is_ming_univision, MingUniVisionConfig)]


def config_from_pretrained(path):
    """-> (registry name, configuration) of the model in `path` (a directory with config.json, or the file itself)."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    with open(path) as f:
        d = json.load(f)
    for name, match, klass in MODEL_REGISTRY:
        if match(d):
            return name, klass.from_dict(d)
    raise ValueError(f"{path}: no model of this framework matches (architecture = {d.get('architecture')!r}, "
                     f"model_type = {d.get('model_type')!r}); known: {[n for n, _, _ in MODEL_REGISTRY]}")
