"""Zuzenex in plain float64 on the CPU: one function per mechanism, whole sequences at a time, no cache and no code shared with the
package.  The tests hold the served path (native step function, arenas, recurrent states, kernels) against it.

A model is (cfg, sd): cfg the dict of a config.json, sd {tensor name: torch tensor}.  Notation: x [T, width] is the residual stream of
one sequence whose first row is position 0.

    layer        h = RMS(x) w1;  x <- x + mixer(h) + ff(h)            (both sublayers read the same normed rows)
    attention    q, k RMS-normed per head with a weight; q_t scaled by 1 + coef ln(floor((t + 1) / every) + 1); causal softmax
                 whose denominator also holds exp(sink_h)
    lightning    S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t with q, k, v = silu(W h); RMS over the joined heads, times
                 sigmoid(W_g h)
    ff           relu(W_up h)^2 through W_down; or a mixture of such experts chosen by softmax scores plus a correction, some of
                 the router's outputs standing for "pass h through", plus an always-on shared expert
"""
import math

import torch

F64 = torch.float64


def f64(t):
    return t.detach().to("cpu", F64)


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(x):
    return x * torch.sigmoid(x)


def relu2(x):
    return torch.relu(x) ** 2


def query_temperature(T, q_temp, pos0=0):
    """[T] factors of the queries at positions pos0 .. pos0 + T - 1."""
    if not q_temp:
        return torch.ones(T, dtype=F64)
    p = torch.arange(pos0, pos0 + T, dtype=torch.int64)
    return 1.0 + float(q_temp["coef"]) * torch.log(torch.div(p + 1, int(q_temp["every"]), rounding_mode="floor").to(F64) + 1.0)


def sink_softmax_attention(q, k, v, sink, scale):
    """q [T, H, d], k [T, G, d], v [T, G, e], sink [H] -> [T, H, e].  Position i sees j <= i; the sink adds exp(sink_h) to the
    denominator and nothing to the numerator."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    for h in range(H):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, -math.inf)
        m = torch.maximum(s.max(-1).values, sink[h])
        p = torch.exp(s - m[:, None])
        den = p.sum(-1) + torch.exp(sink[h] - m)
        out[:, h] = (p @ v[:, g]) / den[:, None]
    return out


def attention_mixer(h, sd, p, m, eps):
    H, G, d, e = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = (h @ f64(sd[p + "q"]).T).reshape(T, H, d)
    k = (h @ f64(sd[p + "k"]).T).reshape(T, G, d)
    v = (h @ f64(sd[p + "v"]).T).reshape(T, G, e)
    q = rms_norm(q, f64(sd[p + "q.norm"]), eps)
    k = rms_norm(k, f64(sd[p + "k.norm"]), eps)
    q = q * query_temperature(T, m.get("q_temp"))[:, None, None]
    o = sink_softmax_attention(q, k, v, f64(sd[p + "sink"]), float(m["scale"]))
    return o.reshape(T, H * e) @ f64(sd[p + "o"]).T


def lightning_recurrence(q, k, v, decay, S0=None):
    """q, k [T, H, d], v [T, H, e], decay [H] -> ([T, H, e], final state [H, d, e]); the state starts at zero (or S0)."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=F64) if S0 is None else S0.clone()
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    return out, S


def lightning_mixer(h, sd, p, m, eps):
    H, d, e = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = silu(h @ f64(sd[p + "q"]).T).reshape(T, H, d)
    k = silu(h @ f64(sd[p + "k"]).T).reshape(T, H, d)
    v = silu(h @ f64(sd[p + "v"]).T).reshape(T, H, e)
    o, _ = lightning_recurrence(q, k, v, torch.tensor([float(a) for a in m["decay"]], dtype=F64))
    o = rms_norm(o.reshape(T, H * e), f64(sd[p + "norm"]), eps) * torch.sigmoid(h @ f64(sd[p + "g"]).T)
    return o @ f64(sd[p + "o"]).T


def expert(h, up, down):
    return relu2(h @ f64(up).T) @ f64(down).T


def route(h, router_w, correction, top):
    """-> (indices [T, top], weights [T, top], scores [T, n]): softmax over every router output, the pick by score + correction,
    the weights from the scores alone."""
    s = torch.softmax(h @ f64(router_w).T, -1)
    idx = torch.topk(s + f64(correction), top, dim=-1).indices
    w = torch.gather(s, 1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20), s


def feed_forward(h, sd, p, mlp):
    if mlp["kind"] == "dense":
        return expert(h, sd[p + "up"], sd[p + "down"])
    r = mlp["router"]
    E, top = int(r["experts"]), int(r["top"])
    idx, w, _ = route(h, sd[p + "router"], sd[p + "correction"], top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            i = int(idx[t, j])
            y = expert(h[t:t + 1], sd[f"{p}e{i}.up"], sd[f"{p}e{i}.down"])[0] if i < E else h[t]      # the outputs past the experts pass h through
            out[t] += w[t, j] * y
    if mlp.get("shared"):
        out = out + expert(h, sd[p + "shared.up"], sd[p + "shared.down"])
    return out


def run_order(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg, sd, tokens, trace=False):
    """-> logits [T, vocab] (and the residual stream after every layer run [runs, T, width])."""
    eps = float(cfg["norm"]["eps"])
    x = f64(sd["embed"])[torch.as_tensor(tokens, dtype=torch.long)]
    streams = []
    for i in run_order(cfg):
        ly = cfg["layers"][i]
        h = rms_norm(x, f64(sd[f"l{i}.norm1"]), eps)
        mixer = {"attention": attention_mixer, "lightning": lightning_mixer}[ly["type"]]
        y = mixer(h, sd, f"l{i}.mix.", ly["mixer"], eps)
        if ly.get("mlp") is not None:
            y = y + feed_forward(h, sd, f"l{i}.mlp.", ly["mlp"])
        x = x + y
        streams.append(x)
    logits = rms_norm(x, f64(sd["final.norm"]), eps) @ f64(sd["head"]).T
    return (logits, torch.stack(streams)) if trace else logits


# ---- small models for the tests ------------------------------------------------------------------------------------------------
def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.25, q_temp=(0.4, 8), mlp=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def lightning_layer(heads=4, dim=16, vdim=16, decay=None, mlp=None):
    decay = decay if decay is not None else [1.0 - 0.45 / (1 + 2 * h) for h in range(heads)]
    return {"type": "lightning", "mixer": dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)), "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=0, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if identity:
        m["router"]["identity"] = identity
    if shared:
        m["shared"] = {"ff": shared}
    return m


def small_config(layers, width=64, vocab=80, loop=None, eps=1e-5):
    cfg = {"architecture": "Zuzenex", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def param_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    s = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    for i, ly in enumerate(cfg["layers"]):
        p, m, mlp = f"l{i}.", ly["mixer"], ly.get("mlp")
        H, d, e = m["heads"], m["dim"], m["vdim"]
        G = m["kv_heads"] if ly["type"] == "attention" else H
        s.update({p + "norm1": (W,), p + "mix.q": (H * d, W), p + "mix.k": (G * d, W), p + "mix.v": (G * e, W), p + "mix.o": (W, H * e)})
        if ly["type"] == "attention":
            s.update({p + "mix.q.norm": (d,), p + "mix.k.norm": (d,), p + "mix.sink": (H,)})
        else:
            s.update({p + "mix.g": (H * e, W), p + "mix.norm": (H * e,)})
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            s.update({p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
            continue
        r = mlp["router"]
        n = r["experts"] + r.get("identity", 0)
        for j in range(r["experts"]):
            s.update({f"{p}mlp.e{j}.up": (mlp["expert"]["ff"], W), f"{p}mlp.e{j}.down": (W, mlp["expert"]["ff"])})
        s.update({p + "mlp.router": (n, W), p + "mlp.correction": (n,)})
        if mlp.get("shared"):
            s.update({p + "mlp.shared.up": (mlp["shared"]["ff"], W), p + "mlp.shared.down": (W, mlp["shared"]["ff"])})
    return s


def random_weights(cfg, seed=0):
    """bf16 tensors under the checkpoint's names: norm weights around 1, sinks of deviation 1, corrections large enough to change picks."""
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for k, shp in param_shapes(cfg).items():
        r = torch.randn(shp, generator=g)
        if k == "embed":
            t = r
        elif "norm" in k:
            t = 1.0 + 0.1 * r
        elif k.endswith("sink"):
            t = r
        elif k.endswith("correction"):
            t = 0.05 * r
        elif k.endswith("router"):
            t = 2.0 * r * shp[-1] ** -0.5
        else:
            t = 1.3 * r * shp[-1] ** -0.5
        sd[k] = t.to(torch.bfloat16)
    return sd
