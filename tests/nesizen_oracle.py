"""A plain, slow float64 implementation of the Nesizen design, one function per mechanism, written
from the design's equations and sharing no code with butterfly_amd. Tests compare the framework
(CPU reference ops and HIP kernels, caches, scheduler) against it.

Notation: h [T, W] is a sublayer input, weights are stored [out, in] and applied as h @ W.T;
positions count from 0; a whole sequence is always processed from its first token.
"""
import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x divided by its root mean square (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_zero_centered(x, w, eps):
    """RMS norm whose weight is stored around zero: unit(x) * (1 + w)."""
    return rms_unit(x, eps) * (1.0 + w)


def streams_read(xs, w_in):
    """Hyper-connection input: u = sum_s in[s] x_s.  xs [S, T, W]."""
    return torch.einsum("s,stw->tw", w_in, xs)


def streams_write(xs, y, mix, w_out):
    """All streams at once from the old ones: x_t <- sum_s mix[s, t] x_s + out[t] y."""
    S = xs.shape[0]
    new = torch.zeros_like(xs)
    for t in range(S):
        for s in range(S):
            new[t] += mix[s, t] * xs[s]
        new[t] += w_out[t] * y
    return new


def rotate_pairs(x, pos, dims, base):
    """Rotary on the first `dims` dimensions of every head of x [T, H, D]: dimension 2i pairs with
    2i+1, angle pos * base^(-2i/dims)."""
    x = x.clone()
    for i in range(dims // 2):
        ang = pos.to(F64) * base ** (-2.0 * i / dims)
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        u, v = x[:, :, 2 * i].clone(), x[:, :, 2 * i + 1].clone()
        x[:, :, 2 * i] = u * c - v * s
        x[:, :, 2 * i + 1] = v * c + u * s
    return x


def visible(i, j, window, keep_first):
    return j <= i and (i - j < window or j < keep_first)


def window_sink_attention(q, k, v, scale, window, keep_first, sink):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] of one sequence (already rotated). Softmax over the
    visible keys plus a sink term exp(sink_h) that only enlarges the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            js = [j for j in range(T) if visible(i, j, window, keep_first)]
            sc = (k[js, g] @ q[i, h]) * scale
            m = torch.maximum(sc.max(), sink[h])
            e = torch.exp(sc - m)
            den = e.sum() + torch.exp(sink[h] - m)
            out[i, h] = (e / den) @ v[js, g]
    return out


def gated_linear_attention(q, k, v, alpha, state=None):
    """Per head S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t. q (already scaled), k,
    alpha [T, H, D]; v [T, H, Dv]. Returns (o [T, H, Dv], final state [H, D, Dv])."""
    T, H, D = q.shape
    Dv = v.shape[2]
    S = torch.zeros(H, D, Dv, dtype=F64) if state is None else state.clone()
    o = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        for h in range(H):
            S[h] = alpha[t, h][:, None] * S[h] + torch.outer(k[t, h], v[t, h])
            o[t, h] = S[h].T @ q[t, h]
    return o, S


def squared_relu(x):
    return torch.clamp(x, min=0.0) ** 2


def clamped_glu_expert(h, w_gate, w_up, w_down, limit):
    g = torch.clamp(h @ w_gate.T, max=limit)
    u = torch.clamp(h @ w_up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


def sigmoid_router(h, w_router, top):
    """Scores sigmoid(W h); the `top` largest are chosen; weights are the scores themselves."""
    s = torch.sigmoid(h @ w_router.T)
    idx = torch.argsort(s, dim=-1, descending=True, stable=True)[:, :top]
    return idx, torch.gather(s, 1, idx)


def moe_layer(h, W, pre, spec):
    idx, wts = sigmoid_router(h, W[pre + "router"], spec["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wts[t]):
            ep = f"{pre}e{e}."
            out[t] += clamped_glu_expert(w * h[t], W[ep + "gate"], W[ep + "up"], W[ep + "down"], spec["expert"]["limit"])
    return out


def attention_mixer(h, W, p, m, pos, shared):
    """`shared`: {layer: (k, v)} of the layers that have their own keys; a layer with kv_from reads
    from there with its own queries, mask, sink and output projection."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = rotate_pairs((h @ W[p + "q"].T).view(T, H, D), pos, m["rot"]["dims"], m["rot"]["base"])
    if m.get("kv_from") is not None:
        k, v = shared[m["kv_from"]]
    else:
        k = rotate_pairs((h @ W[p + "k"].T).view(T, G, D), pos, m["rot"]["dims"], m["rot"]["base"])
        v = (h @ W[p + "v"].T).view(T, G, Dv)
    o = window_sink_attention(q, k, v, m["scale"], m["mask"]["size"], m["mask"].get("keep_first", 0), W[p + "sink"])
    return o.reshape(T, H * Dv) @ W[p + "o"].T, (k, v)


def gla_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, Dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = torch.sigmoid(z).view(T, H, D) ** (1.0 / m["tau"])
    o, _ = gated_linear_attention(q, k, v, alpha)
    o = rms_unit(o, eps) * W[p + "norm"]
    gate = h @ W[p + "g"].T
    return (o.reshape(T, H * Dv) * (gate * torch.sigmoid(gate))) @ W[p + "o"].T


def forward(cfg, weights, tokens, layer_outputs=None):
    """Logits [T, vocab] of one whole sequence. cfg: the config.json dict; weights: tensors by
    their checkpoint names."""
    W = {n: t.to(F64) for n, t in weights.items()}
    eps, S, T = cfg["norm"]["eps"], cfg["streams"], len(tokens)
    pos = torch.arange(T)
    x0 = norm_zero_centered(W["embed"][torch.tensor(tokens)], W["embed.norm"], eps)
    xs = torch.stack([x0.clone() for _ in range(S)])
    shared = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = norm_zero_centered(streams_read(xs, W[p + "hc1.in"]), W[p + "norm1"], eps)
        if L["type"] == "attention":
            y, kv = attention_mixer(h, W, p + "mix.", L["mixer"], pos, shared)
            if L["mixer"].get("kv_from") is None:
                shared[i] = kv
        else:
            y = gla_mixer(h, W, p + "mix.", L["mixer"], eps)
        xs = streams_write(xs, y, W[p + "hc1.mix"], W[p + "hc1.out"])
        if L.get("mlp") is not None:
            h = norm_zero_centered(streams_read(xs, W[p + "hc2.in"]), W[p + "norm2"], eps)
            if L["mlp"]["kind"] == "dense":
                y = squared_relu(h @ W[p + "mlp.up"].T) @ W[p + "mlp.down"].T
            else:
                y = moe_layer(h, W, p + "mlp.", L["mlp"])
            xs = streams_write(xs, y, W[p + "hc2.mix"], W[p + "hc2.out"])
        if layer_outputs is not None:
            layer_outputs.append(xs.sum(0))
    return norm_zero_centered(xs.sum(0), W["final.norm"], eps) @ W["head"].T


def greedy(cfg, weights, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]


# ---------------------------------------------------------------------------------------
# random models for the tests
# ---------------------------------------------------------------------------------------
def random_weights(cfg, seed, decay_rank=3):
    """Random bf16-representable weights for `cfg`, by checkpoint name."""
    g = torch.Generator().manual_seed(seed)
    W, S, Wd = {}, cfg["streams"], cfg["width"]

    def rnd(*shape, std=None, mean=0.0):
        std = (1.0 / math.sqrt(shape[-1])) if std is None else std
        return (mean + std * torch.randn(*shape, generator=g)).to(torch.bfloat16)

    W["embed"] = rnd(cfg["vocab"], Wd, std=1.0)
    W["embed.norm"] = rnd(Wd, std=0.2)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        subl = ("1", "2") if L.get("mlp") is not None else ("1",)
        for q in subl:
            W[p + f"norm{q}"] = rnd(Wd, std=0.2)
            W[p + f"hc{q}.in"] = rnd(S, std=0.2, mean=1.0 / S)
            W[p + f"hc{q}.out"] = rnd(S, std=0.2, mean=1.0)
            W[p + f"hc{q}.mix"] = (torch.eye(S) + 0.15 * torch.randn(S, S, generator=g)).to(torch.bfloat16)
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        if L["type"] == "attention":
            G = m.get("kv_heads", H)
            W[p + "mix.q"] = rnd(H * D, Wd, std=2.0 / math.sqrt(Wd))
            if m.get("kv_from") is None:
                W[p + "mix.k"] = rnd(G * D, Wd, std=2.0 / math.sqrt(Wd))
                W[p + "mix.v"] = rnd(G * Dv, Wd)
            W[p + "mix.sink"] = rnd(H, std=1.0)
        else:
            W[p + "mix.q"], W[p + "mix.k"] = rnd(H * D, Wd), rnd(H * D, Wd)
            W[p + "mix.v"], W[p + "mix.g"] = rnd(H * Dv, Wd), rnd(H * Dv, Wd)
            W[p + "mix.a1"], W[p + "mix.a2"] = rnd(decay_rank, Wd), rnd(H * D, decay_rank, std=1.0)
            W[p + "mix.a2.b"] = rnd(H * D, std=1.0, mean=2.0)
            W[p + "mix.norm"] = rnd(Dv, std=0.2, mean=1.0)
        W[p + "mix.o"] = rnd(Wd, H * Dv)
        f = L.get("mlp")
        if f is None:
            continue
        if f["kind"] == "dense":
            W[p + "mlp.up"], W[p + "mlp.down"] = rnd(f["ff"], Wd), rnd(Wd, f["ff"])
        else:
            W[p + "mlp.router"] = rnd(f["router"]["experts"], Wd, std=2.0 / math.sqrt(Wd))
            for e in range(f["router"]["experts"]):
                W[p + f"mlp.e{e}.gate"] = rnd(f["expert"]["ff"], Wd, std=2.0 / math.sqrt(Wd))
                W[p + f"mlp.e{e}.up"] = rnd(f["expert"]["ff"], Wd, std=2.0 / math.sqrt(Wd))
                W[p + f"mlp.e{e}.down"] = rnd(Wd, f["expert"]["ff"])
    W["final.norm"] = rnd(Wd, std=0.2)
    W["head"] = rnd(cfg["vocab"], Wd)
    return W


def attn_layer(heads, kv_heads, dim, vdim, rot, base, scale, window, keep_first, mlp, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": {"dims": rot, "base": base},
         "scale": scale, "mask": {"size": window, "keep_first": keep_first}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def gla_layer(heads, dim, vdim, tau, mlp):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def config(layers, width, vocab, streams, eps=1e-5):
    return {"architecture": "Nesizen", "layers": layers, "norm": {"eps": eps}, "streams": streams, "vocab": vocab,
            "width": width}
