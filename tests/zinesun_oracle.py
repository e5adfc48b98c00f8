"""A plain, slow float64 implementation of the Zinesun design, one function per mechanism, written
from the design's equations and sharing no code with the package. Keys and values are expanded
per head from the cached latent (the package never does that), every loop is explicit where it
makes the definition plainer. Tests build configurations and random weights here."""
import math

import torch

F64 = torch.float64


# ---- configuration builders ----------------------------------------------------------------
def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, q_rank, base, scale, window, mlp):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "rot": {"base": base, "dims": rot_dim}, "scale": scale, "mask": {"size": window}}}


def config(layers, width, vocab, eps, taps, embed_scale):
    return {"architecture": "Zinesun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps},
            "embedding": {"scale": embed_scale}, "layers": layers}


def random_weights(cfg, seed):
    """name -> bf16 tensor, under the names a model folder uses."""
    g = torch.Generator().manual_seed(seed)
    W, out = cfg["width"], {}

    def mat(name, rows, cols, std=None):
        out[name] = (torch.randn(rows, cols, generator=g) * (std or 1.0 / math.sqrt(cols))).to(torch.bfloat16)

    def vec(name, n, mean, std):
        out[name] = (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    mat("embed", cfg["vocab"], W, 1.0 / max(cfg["embedding"]["scale"], 1e-3))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, D, rd, Dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        for n in ("norm1", "norm2") if L["mlp"] else ("norm1",):
            vec(p + n, W, 1.0, 0.2)
            vec(p + n + ".b", W, 0.0, 0.2)
        vec(p + "ls1", W, 0.6, 0.2)
        if L["mlp"]:
            vec(p + "ls2", W, 0.6, 0.2)
        if cfg["canon"]["taps"] > 0:
            mat(p + "canon1", W, cfg["canon"]["taps"], 0.4)
        out[p + "dwa"] = (torch.randn(i + 2, generator=g) * 0.3 + torch.tensor([0.0] * (i + 1) + [0.7])).to(torch.bfloat16)
        mat(p + "mix.dq", Q, W)
        vec(p + "mix.dq.norm", Q, 1.0, 0.2)
        mat(p + "mix.uq", H * (D + rd), Q)
        mat(p + "mix.dkv", R + rd, W)
        vec(p + "mix.dkv.norm", R, 1.0, 0.2)
        mat(p + "mix.uk", H * D, R)
        mat(p + "mix.uv", H * Dv, R)
        mat(p + "mix.g", H, W)
        mat(p + "mix.o", W, H * Dv)
        f = L["mlp"]
        if f and f["kind"] == "dense":
            mat(p + "mlp.up", f["ff"], W)
            mat(p + "mlp.down", W, f["ff"])
            vec(p + "mlp.act", 2, 0.0, 1.0)
        elif f:
            E, F = f["router"]["experts"], f["expert"]["ff"]
            mat(p + "mlp.router", E, W, 2.0 / math.sqrt(W))
            vec(p + "mlp.router.b", E, 0.0, 0.5)
            for e in range(E):
                mat(p + f"mlp.e{e}.gate", F, W)
                mat(p + f"mlp.e{e}.up", F, W)
                mat(p + f"mlp.e{e}.down", W, F)
    vec("final.norm", W, 1.0, 0.2)
    vec("final.norm.b", W, 0.0, 0.2)
    return out


# ---- mechanisms -----------------------------------------------------------------------------
def scaled_embedding(table, tokens, scale):
    return table[torch.tensor(tokens)] * scale


def causal_conv_residual(x, w):
    """x [T, C], w [C, taps]: out_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j), zeros before t = 0."""
    T, taps = x.shape[0], w.shape[1]
    out = x.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * x[s]
    return out


def layer_norm(y, w, b, eps):
    mu = y.mean(-1, keepdim=True)
    var = ((y - mu) ** 2).mean(-1, keepdim=True)
    return (y - mu) / torch.sqrt(var + eps) * w + b


def rms_norm(y, w, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * w


def rotate_pairs(v, position, base, dims):
    """v [..., n]: the pairs (2i, 2i+1), i < dims / 2, turned by position * base^(-2i / dims)."""
    out = v.clone()
    for i in range(dims // 2):
        a = position * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        out[..., 2 * i] = v[..., 2 * i] * c - v[..., 2 * i + 1] * s
        out[..., 2 * i + 1] = v[..., 2 * i + 1] * c + v[..., 2 * i] * s
    return out


def windowed_softmax_attention(q, k, v, scale, window):
    """q, k [T, D], v [T, Dv] of one head: row i sees j with 0 <= i - j < window."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for i in range(T):
        lo = max(0, i - window + 1)
        s = (k[lo:i + 1] @ q[i]) * scale
        out[i] = torch.softmax(s, 0) @ v[lo:i + 1]
    return out


def latent_attention(h, P, m, eps):
    """h [T, W]; P: the mixer's tensors by short name; m: its config entry."""
    T = h.shape[0]
    H, D, rd, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ P["dq"].T, P["dq.norm"], eps)
    q = (cq @ P["uq"].T).view(T, H, D + rd)
    dkv = h @ P["dkv"].T
    c = rms_norm(dkv[:, :R], P["dkv.norm"], eps)
    k_rot = torch.stack([rotate_pairs(dkv[t, R:], t, m["rot"]["base"], m["rot"]["dims"]) for t in range(T)])
    k_plain = (c @ P["uk"].T).view(T, H, D)
    val = (c @ P["uv"].T).view(T, H, Dv)
    gate = torch.sigmoid(h @ P["g"].T)
    heads = []
    for hd in range(H):
        q_rot = torch.stack([rotate_pairs(q[t, hd, D:], t, m["rot"]["base"], m["rot"]["dims"]) for t in range(T)])
        qh = torch.cat([q[:, hd, :D], q_rot], 1)
        kh = torch.cat([k_plain[:, hd], k_rot], 1)
        o = windowed_softmax_attention(qh, kh, val[:, hd], m["scale"], m["mask"]["size"])
        heads.append(o * gate[:, hd:hd + 1])
    return torch.cat(heads, 1) @ P["o"].T


def softplus(v):
    return math.log1p(math.exp(-abs(v))) + max(v, 0.0)


def xielu(z, p, q):
    pos = softplus(p) * z * z + z / 2
    neg = (0.5 + softplus(q)) * (torch.expm1(z) - z) + z / 2
    return torch.where(z > 0, pos, neg)


def dense_ffn(x, up, down, act):
    return xielu(x @ up.T, float(act[0]), float(act[1])) @ down.T


def route(x, router, bias, top):
    """-> chosen experts [T, top], weights [T, top]: the softmax over the chosen logits only."""
    logits = x @ router.T + bias
    val, idx = torch.topk(logits, top, -1)
    return idx, torch.softmax(val, -1)


def moe_ffn(x, P, experts, top):
    idx, w = route(x, P["router"], P["router.b"], top)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            g, u = P[f"e{e}.gate"] @ x[t], P[f"e{e}.up"] @ x[t]
            out[t] += w[t, j] * (P[f"e{e}.down"] @ (g * torch.sigmoid(g) * u))
    return out


def depth_average(results, weights):
    return sum(weights[j] * results[j] for j in range(len(results)))


def _sub(W, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in W.items() if k.startswith(prefix)}


def forward(cfg, W, tokens, layer_out=None):
    """Logits [T, vocab] of one sequence; layer_out (a list) collects what every layer hands on."""
    eps = cfg["norm"]["eps"]
    table = W["embed"].to(F64)
    x = scaled_embedding(table, tokens, cfg["embedding"]["scale"])
    results = [x]
    for i, L in enumerate(cfg["layers"]):
        P = _sub(W, f"l{i}.")
        h = causal_conv_residual(x, P["canon1"]) if cfg["canon"]["taps"] > 0 else x
        y = latent_attention(h, _sub(W, f"l{i}.mix."), L["mixer"], eps)
        x = x + P["ls1"] * layer_norm(y, P["norm1"], P["norm1.b"], eps)
        f = L["mlp"]
        if f is not None:
            M = _sub(W, f"l{i}.mlp.")
            y = dense_ffn(x, M["up"], M["down"], M["act"]) if f["kind"] == "dense" else \
                moe_ffn(x, M, f["router"]["experts"], f["router"]["top"])
            x = x + P["ls2"] * layer_norm(y, P["norm2"], P["norm2.b"], eps)
        results.append(x)
        x = depth_average(results, P["dwa"])
        if layer_out is not None:
            layer_out.append(x)
    x = layer_norm(x, W["final.norm"].to(F64), W["final.norm.b"].to(F64), eps)
    return x @ table.T


def greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]
