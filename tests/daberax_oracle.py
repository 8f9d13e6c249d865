"""Daberax in plain float64 on the CPU: one function per mechanism, whole sequences at a time, no cache and no code shared with the
package.  The tests hold the served path (native step function, arenas, recurrent states, kernels) against it.

A model is (cfg, sd): cfg the dict of a config.json, sd {tensor name: torch tensor}.  Notation: x [T, width] is the residual stream of
one sequence whose first row is position 0; rms(y) = y / sqrt(mean(y^2) + eps).

    layer        x <- x + w1 rms(mixer(x));  x <- x + w2 rms(ff(x));  x <- x + ws rms(P (gelu(G x) * e_tok))      (the norm sits on
                 every sublayer's RESULT; the sublayers read x as it is; the last term takes a slice of a second embedding table)
    delta        gated delta rule on conv'd, silu'd, unit-length q / k:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    attention    grouped heads, biases, RMS over the WHOLE q and k projections, interleaved rotary pairs with optional long-context
                 frequency scaling, optional tanh soft cap of the scores, optional sliding window, one sigmoid gate per head
    latent       keys and values of all heads are linear maps of one normed latent per token; a rotated key part is shared by the heads
    ff           W_down (gelu(W_gate x) * (W_up x)),  gelu in its tanh form
"""
import math

import torch

F64 = torch.float64


def f64(t):
    return t.detach().to("cpu", F64)


def rms(y, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ---- positions -----------------------------------------------------------------------------------------------------------------
def rotary_frequencies(rot):
    """[dims / 2] angles per position: base^(-2i / dims), optionally rescaled by wavelength (short waves kept, long waves divided by
    `factor`, a linear blend between)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc:
        fac, lo, hi, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for fi in f:
            wave = 2.0 * math.pi / fi
            if wave < orig / hi:
                out.append(fi)
            elif wave > orig / lo:
                out.append(fi / fac)
            else:
                s = (orig / wave - lo) / (hi - lo)
                out.append((1.0 - s) * fi / fac + s * fi)
        f = out
    return torch.tensor(f, dtype=F64)


def rotate_interleaved(x, freq, pos0=0):
    """x [T, ..., n]: values (2i, 2i + 1), i < len(freq), of the last axis turn by the angle position * freq_i; the rest pass."""
    T = x.shape[0]
    n = 2 * freq.numel()
    ang = torch.arange(pos0, pos0 + T, dtype=F64)[:, None] * freq[None, :]
    shape = [T] + [1] * (x.dim() - 2) + [n // 2]
    c, s = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    a, b = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = a * c - b * s
    out[..., 1:n:2] = b * c + a * s
    return out


def visible(T, window):
    """[T, T] mask: row i sees column j when 0 <= i - j (< window, if there is one)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if window:
        m &= (i - j) < int(window)
    return m


def masked_softmax_attention(q, k, v, scale, window=None, softcap=None):
    """q [T, H, d], k [T, G, d], v [T, G, e] -> [T, H, e]; query head h reads key/value head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    mask = visible(T, window)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~mask, -math.inf)
        out[:, h] = torch.softmax(s, -1) @ v[:, g]
    return out


# ---- mixers --------------------------------------------------------------------------------------------------------------------
def attention_mixer(h, sd, p, m, eps):
    H, G, d, e = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = h @ f64(sd[p + "q"]).T + f64(sd[p + "q.b"])
    k = h @ f64(sd[p + "k"]).T + f64(sd[p + "k.b"])
    v = h @ f64(sd[p + "v"]).T + f64(sd[p + "v.b"])
    q = (rms(q, eps) * f64(sd[p + "q.norm"])).reshape(T, H, d)
    k = (rms(k, eps) * f64(sd[p + "k.norm"])).reshape(T, G, d)
    if m.get("rot"):
        fr = rotary_frequencies(m["rot"])
        q, k = rotate_interleaved(q, fr), rotate_interleaved(k, fr)
    o = masked_softmax_attention(q, k, v.reshape(T, G, e), float(m["scale"]), (m.get("mask") or {}).get("size"), m.get("softcap"))
    gate = torch.sigmoid(h @ f64(sd[p + "g"]).T)                       # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * e) @ f64(sd[p + "o"]).T + f64(sd[p + "o.b"])


def latent_attention_mixer(h, sd, p, m, eps):
    H, d, r, e, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    T = h.shape[0]
    q = (h @ f64(sd[p + "q"]).T).reshape(T, H, d + r)
    dkv = h @ f64(sd[p + "dkv"]).T
    c = rms(dkv[:, :R], eps) * f64(sd[p + "dkv.norm"])
    kr = dkv[:, R:].reshape(T, 1, r)
    fr = rotary_frequencies(m["rot"])
    assert 2 * fr.numel() == r
    q_rot = rotate_interleaved(q[:, :, d:].contiguous(), fr)
    kr = rotate_interleaved(kr, fr)
    kn = (c @ f64(sd[p + "uk"]).T).reshape(T, H, d)
    v = (c @ f64(sd[p + "uv"]).T).reshape(T, H, e)
    qq = torch.cat([q[:, :, :d], q_rot], -1)
    kk = torch.cat([kn, kr.expand(T, H, r)], -1)
    o = masked_softmax_attention(qq, kk, v, float(m["scale"]), (m.get("mask") or {}).get("size"), m.get("softcap"))
    return o.reshape(T, H * e) @ f64(sd[p + "o"]).T


def causal_conv(x, w):
    """x [T, C], w [C, taps] (last column multiplies the current row, zeros before the start) -> [T, C]."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], 0)
    out = torch.zeros(T, C, dtype=F64)
    for j in range(taps):
        out += pad[j:j + T] * w[:, j]
    return out


def gated_delta_rule(q, k, v, beta, g, S0=None):
    """q, k [T, H, d], v [T, H, e], beta, g [T, H] -> ([T, H, e], final state [H, d, e])."""
    T, H, d = q.shape
    e = v.shape[2]
    S = torch.zeros(H, d, e, dtype=F64) if S0 is None else S0.clone()
    out = torch.zeros(T, H, e, dtype=F64)
    for t in range(T):
        S = S * g[t][:, None, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hde,hd->he", S, k[t]))
        S = S + torch.einsum("hd,he->hde", k[t], u)
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    return out, S


def delta_mixer(h, sd, p, m, eps):
    H, G, d, e = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = silu(causal_conv(h @ f64(sd[p + "q"]).T, f64(sd[p + "q.conv"]))).reshape(T, G, d)
    k = silu(causal_conv(h @ f64(sd[p + "k"]).T, f64(sd[p + "k.conv"]))).reshape(T, G, d)
    v = silu(causal_conv(h @ f64(sd[p + "v"]).T, f64(sd[p + "v.conv"]))).reshape(T, H, e)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(h @ f64(sd[p + "b"]).T)
    g = torch.exp(-torch.exp(f64(sd[p + "A_log"])) * softplus(h @ f64(sd[p + "a"]).T + f64(sd[p + "dt_bias"])))
    o, _ = gated_delta_rule(q, k, v, beta, g)
    o = rms(o, eps) * f64(sd[p + "norm"])
    o = o * silu(h @ f64(sd[p + "g"]).T).reshape(T, H, e)
    return o.reshape(T, H * e) @ f64(sd[p + "o"]).T


MIXERS = {"attention": attention_mixer, "latent_attention": latent_attention_mixer, "delta": delta_mixer}


# ---- the stack -----------------------------------------------------------------------------------------------------------------
def dense_ff(x, sd, p):
    return (gelu_tanh(x @ f64(sd[p + "gate"]).T) * (x @ f64(sd[p + "up"]).T)) @ f64(sd[p + "down"]).T


def token_side(x, tokens, sd, i, side_dim, eps):
    e = f64(sd["side.embed"])[tokens][:, i * side_dim:(i + 1) * side_dim]
    y = (gelu_tanh(x @ f64(sd[f"l{i}.side.gate"]).T) * e) @ f64(sd[f"l{i}.side.proj"]).T
    return rms(y, eps) * f64(sd[f"l{i}.side.norm"])


def forward(cfg, sd, tokens):
    """tokens: list of ids of one sequence -> (logits [T, vocab], residual streams after every layer [layers, T, width])."""
    eps = float(cfg["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = f64(sd["embed"])[tokens]
    side = cfg.get("token_side")
    streams = []
    for i, ly in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + rms(MIXERS[ly["type"]](x, sd, p + "mix.", ly["mixer"], eps), eps) * f64(sd[p + "norm1"])
        if ly.get("mlp") is not None:
            x = x + rms(dense_ff(x, sd, p + "mlp."), eps) * f64(sd[p + "norm2"])
        if side:
            x = x + token_side(x, tokens, sd, i, int(side["dim"]), eps)
        streams.append(x)
    y = rms(x, eps) * f64(sd["final.norm"])
    return (y @ f64(sd["head"]).T) * float(cfg.get("logit_scale", 1.0)), torch.stack(streams)


# ---- small models for the tests ----------------------------------------------------------------------------------------------------
def dense(ff):
    return {"kind": "dense", "ff": ff}


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.25, rot=(10000.0, 16), scaling=None, softcap=None, window=None, mlp=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if softcap:
        m["softcap"] = softcap
    if window:
        m["mask"] = {"size": window}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent_layer(heads=4, dim=8, rot_dim=8, vdim=12, kv_rank=24, scale=0.25, base=10000.0, softcap=None, window=None, mlp=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale, rot={"base": base, "dims": rot_dim})
    if softcap:
        m["softcap"] = softcap
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def delta_layer(heads=4, kv_heads=2, dim=16, vdim=16, conv=4, mlp=None):
    return {"type": "delta", "mixer": dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv), "mlp": mlp}


def small_config(layers, width=64, vocab=80, side=6, logit_scale=0.5, eps=1e-5):
    cfg = {"architecture": "Daberax", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers, "logit_scale": logit_scale}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


def param_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    side = (cfg.get("token_side") or {}).get("dim", 0)
    s = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    if side:
        s["side.embed"] = (V, side * len(cfg["layers"]))
    for i, ly in enumerate(cfg["layers"]):
        p, m, t = f"l{i}.", ly["mixer"], ly["type"]
        H, d, e = m["heads"], m["dim"], m["vdim"]
        s.update({p + "norm1": (W,), p + "mix.o": (W, H * e)})
        if t == "attention":
            G = m["kv_heads"]
            s.update({p + "mix.q": (H * d, W), p + "mix.k": (G * d, W), p + "mix.v": (G * e, W), p + "mix.q.b": (H * d,), p + "mix.k.b": (G * d,),
                      p + "mix.v.b": (G * e,), p + "mix.o.b": (W,), p + "mix.q.norm": (H * d,), p + "mix.k.norm": (G * d,), p + "mix.g": (H, W)})
        elif t == "latent_attention":
            r, R = m["rot_dim"], m["kv_rank"]
            s.update({p + "mix.q": (H * (d + r), W), p + "mix.dkv": (R + r, W), p + "mix.dkv.norm": (R,), p + "mix.uk": (H * d, R),
                      p + "mix.uv": (H * e, R)})
        else:
            G, taps = m["kv_heads"], m["conv"]
            s.update({p + "mix.q": (G * d, W), p + "mix.k": (G * d, W), p + "mix.v": (H * e, W), p + "mix.q.conv": (G * d, taps),
                      p + "mix.k.conv": (G * d, taps), p + "mix.v.conv": (H * e, taps), p + "mix.b": (H, W), p + "mix.a": (H, W),
                      p + "mix.A_log": (H,), p + "mix.dt_bias": (H,), p + "mix.norm": (e,), p + "mix.g": (H * e, W)})
        if ly.get("mlp") is not None:
            ff = ly["mlp"]["ff"]
            s.update({p + "norm2": (W,), p + "mlp.gate": (ff, W), p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
        if side:
            s.update({p + "side.gate": (side, W), p + "side.proj": (W, side), p + "side.norm": (W,)})
    return s


def random_weights(cfg, seed=0):
    """bf16 tensors under the checkpoint's names: norm weights around 1, decays spread between slow and fast, biases that matter."""
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for k, shp in param_shapes(cfg).items():
        r = torch.randn(shp, generator=g)
        if k in ("embed", "side.embed"):
            t = r
        elif "norm" in k:
            t = 1.0 + 0.1 * r
        elif k.endswith("A_log"):
            t = -1.0 + r
        elif k.endswith("dt_bias"):
            t = r
        elif k.endswith(".conv"):
            t = 0.6 * r
        elif len(shp) == 1:
            t = 0.3 * r
        else:
            t = 1.3 * r * shp[-1] ** -0.5
        sd[k] = t.to(torch.bfloat16)
    return sd
