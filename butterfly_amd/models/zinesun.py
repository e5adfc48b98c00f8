"""Zinesun: a decoder-only LM of latent-attention layers on a post-norm residual (ModelConfig.layer_specs).

  embedding   : x = table[token] * embed_scale, an f32 residual
  every layer : h = x + conv(x)          causal per-channel convolution over time (conv_taps taps,
                                         no bias); the last taps - 1 inputs of every layer live in
                                         the cache's per-sequence state slots
                x <- x + ls1 * LN1(mixer(h))           layer norm (weight, bias) on the sublayer's
                x <- x + ls2 * LN2(ff(x))              OUTPUT, a per-channel scale, then the sum
                X_(i+1) = x;  x <- sum_(j <= i+1) avg_i[j] X_j       X_0 = the embedding output:
                                         what the next layer reads is a learned average over the
                                         results of all layers so far
    mixer "latent_attention" : c_q = rms(W_dq h), q = W_uq c_q (per head [dim | rot_dim]);
                        W_dkv h = [c | k_rot]: c RMS-normed, k_rot rotated (interleaved pairs) and
                        shared by the heads. Only [c | k_rot] is cached. Keys and values are never
                        expanded: the unrotated query part is carried into the latent space
                        (q_lat = W_uk^T q_nope per head), so all heads attend to one shared
                        "key" [c | k_rot] and "value" c (multi-query attention over the latent),
                        and the head's value projection W_uv is applied to the attended latent.
                        Causal sliding window, ordinary softmax, per-head sigmoid output gate.
    feed-forward      : dense W_down xIELU(W_up x), or a router (f32 logits + bias, top-k, softmax
                        over the chosen logits) over plain silu-GLU experts whose outputs are
                        summed with the routing weights
  output      : layer norm, logits = table x (the embedding table, unscaled), f32

Every size and constant comes from the config; the residual, norms, softmax, rotary angles, router
and gates run in f32 in the bf16 model too. Unsharded (tp = pp = ep = 1). Prompt chunks always
attend through the paged cache, so one attention op serves fresh prompts, continuation chunks and
decoded tokens (its kernel forms share one mask rule: which one runs changes a result only by
rounding).
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .. import ops
from ..config import ModelConfig
from ..engine.batch import ForwardBatch
from ..parallel.comm import Communicator
from .shard import LocalDims, Shard
from .stack import PackedStack, pad128
from .transformer import LogicalParam, _name_seed


def _softplus(v: float) -> float:
    return v + math.log1p(math.exp(-v)) if v > 0 else math.log1p(math.exp(v))


class ZinesunLM(PackedStack):
    attention_types = ("latent_attention",)

    def __init__(self, cfg: ModelConfig, shard: Shard = Shard(), device="cpu",
                 dtype: torch.dtype = torch.bfloat16, comm: Optional[Communicator] = None):
        if not cfg.layer_specs:
            raise ValueError("Zinesun needs ModelConfig.layer_specs (ModelConfig.from_zinesun)")
        if shard.tp_size != 1 or shard.ep_size != 1 or shard.layer_start != 0 or \
                (shard.layer_end is not None and shard.layer_end != cfg.num_layers):
            raise NotImplementedError("Zinesun runs unsharded (tp = pp = ep = 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Zinesun runs in bfloat16 or float32")
        for sp in cfg.layer_specs:
            if sp["type"] != "latent_attention":
                raise ValueError(f"layer {sp['index']}: Zinesun has no mixer {sp['type']!r}")
        self.cfg, self.shard = cfg, shard
        self.device, self.dtype = torch.device(device), dtype
        self.comm = comm or Communicator.single()
        self.specs = cfg.layer_specs
        self.taps = int(cfg.conv_taps)
        self.layer_ids = list(range(cfg.num_layers))
        self.first = self.last = True
        self.tp = self.ep = 1
        vpad = pad128(cfg.vocab_size)
        self.dims = LocalDims(hq=cfg.num_heads, hkv=1, kv_head0=0, q_head0=0,
                              ffn=max(cfg.intermediate_size, 1), ffn0=0, vocab=vpad, vocab0=0, vocab_padded=vpad,
                              experts=max(cfg.num_experts, 1), expert0=0)
        self.cache_index = {sp["index"]: n for n, sp in enumerate(self.specs)}
        # cached row widths: [latent | rotated key part] and the latent, padded with zeros to sizes
        # the attention's matrix-core form tiles
        self.cache_dims = [(ops.attn_window_pad(sp["kv_rank"] + sp["rot_dim"], dtype),
                            ops.attn_window_pad(sp["kv_rank"], dtype)) for sp in self.specs]
        self.has_state = self.taps > 1            # the convolution's history
        self.state: list = []                     # set by allocate_state (the cache object owns the pool)
        self.layer_probe = None                   # debug hook: f(layer, residual [T, W] f32) after every layer
        self.p: dict[str, torch.Tensor] = {}
        self.packed: dict = {}
        self._arange: dict = {}
        self._act: dict = {}                      # layer -> xIELU coefficients (floats), from p[...act]
        self._alloc()

    # ------------------------------------------------------------------------------------
    # parameters
    # ------------------------------------------------------------------------------------
    def _wide(self, rows: int, k: int) -> int:
        """Rows of a projection: padded to the tuned GEMMs' 128-row tiling when its K fits them."""
        return pad128(rows) if k % 64 == 0 else rows

    def _alloc(self):
        c, W = self.cfg, self.cfg.hidden_size
        z = lambda *s: torch.zeros(*s, dtype=self.dtype, device=self.device)                  # noqa: E731
        f = lambda *s: torch.zeros(*s, dtype=torch.float32, device=self.device)               # noqa: E731
        p = self.p
        p["embed"] = z(self.dims.vocab, W)            # rows past the vocabulary stay zero (tied LM head)
        for n, sp in enumerate(self.specs):
            pre = f"l{sp['index']}."
            H, D, Dv, R, Q, rd = sp["heads"], sp["dim"], sp["vdim"], sp["kv_rank"], sp["q_rank"], sp["rot_dim"]
            p[pre + "norm1"], p[pre + "norm1.b"], p[pre + "ls1"] = f(W), f(W), f(W)
            if self.taps > 0:
                p[pre + "canon1"] = f(W, self.taps)
            p[pre + "dwa"] = f(n + 2)
            # one projection of the mixer's input: query latent | key/value latent | rotated key | gates
            p[pre + "in"] = z(self._wide(Q + R + rd + H, W), W)
            p[pre + "dq.norm"], p[pre + "dkv.norm"] = f(Q), f(R)
            p[pre + "uq"] = z(self._wide(H * (D + rd), Q), Q)
            p[pre + "ukT"] = z(H, R, D)               # W_uk per head, transposed: q_lat = ukT[h] q_nope
            p[pre + "uv"] = z(H, Dv, R)
            p[pre + "o"] = z(W, H * Dv)
            # frequencies of the rotated pairs of the rot_dim part (its first rot_dims dimensions)
            i = torch.arange(sp["rot_dims"] // 2, dtype=torch.float64)
            p[pre + "inv_freq"] = (sp["rot_base"] ** (-2.0 * i / max(sp["rot_dims"], 1))).to(torch.float32).to(self.device)
            fs = sp["ffn"]
            if fs:
                p[pre + "norm2"], p[pre + "norm2.b"], p[pre + "ls2"] = f(W), f(W), f(W)
                if fs["kind"] == "dense":
                    ffp = self._wide(fs["ff"], W)
                    p[pre + "up"], p[pre + "down"], p[pre + "act"] = z(ffp, W), z(W, ffp), f(2)
                else:
                    E, F = fs["experts"], fs["ff"]
                    p[pre + "router"], p[pre + "router.b"] = z(E, W), f(E)
                    p[pre + "gate_up"], p[pre + "edown"] = z(E, 2 * F, W), z(E, W, F)
        p["final.norm"], p["final.norm.b"] = f(W), f(W)

    @property
    def head_weight(self) -> torch.Tensor:
        return self.p["embed"]

    def logical_params(self) -> list[LogicalParam]:
        """Checkpoint tensors by their file names ('l<i>.mix.dq', 'l<i>.mlp.e<j>.gate', ...), each a
        view into (or a transposition of) the fused local tensors."""
        c, p = self.cfg, self.p
        out: list[LogicalParam] = []

        def add(name, t, init="normal", shape=None, get=None, put=None):
            out.append(LogicalParam(name, tuple(shape or t.shape), None, 0, 0, init, get or (lambda t=t: t),
                                    put or (lambda x, t=t: t.copy_(x.reshape(t.shape)))))

        add("embed", p["embed"][:c.vocab_size], "embed")
        for sp in self.specs:
            i = sp["index"]
            L = f"l{i}."
            H, D, Dv, R, Q, rd = sp["heads"], sp["dim"], sp["vdim"], sp["kv_rank"], sp["q_rank"], sp["rot_dim"]
            add(L + "norm1", p[L + "norm1"], "ones")
            add(L + "norm1.b", p[L + "norm1.b"], "small")
            add(L + "ls1", p[L + "ls1"], "scale")
            if self.taps > 0:
                add(L + "canon1", p[L + "canon1"], "taps")
            add(L + "dwa", p[L + "dwa"], "avg")
            w = p[L + "in"]
            add(L + "mix.dq", w[:Q])
            add(L + "mix.dkv", w[Q:Q + R + rd])
            add(L + "mix.g", w[Q + R + rd:Q + R + rd + H])
            add(L + "mix.dq.norm", p[L + "dq.norm"], "ones")
            add(L + "mix.dkv.norm", p[L + "dkv.norm"], "ones")
            add(L + "mix.uq", p[L + "uq"][:H * (D + rd)])
            ukT, uv = p[L + "ukT"], p[L + "uv"]
            add(L + "mix.uk", ukT, shape=(H * D, R), get=lambda t=ukT: t.transpose(1, 2).reshape(-1, t.shape[1]),
                put=lambda x, t=ukT: t.copy_(x.reshape(t.shape[0], t.shape[2], t.shape[1]).transpose(1, 2)))
            add(L + "mix.uv", uv, shape=(H * Dv, R), get=lambda t=uv: t.reshape(-1, t.shape[2]))
            add(L + "mix.o", p[L + "o"])
            fs = sp["ffn"]
            if fs:
                add(L + "norm2", p[L + "norm2"], "ones")
                add(L + "norm2.b", p[L + "norm2.b"], "small")
                add(L + "ls2", p[L + "ls2"], "scale")
                if fs["kind"] == "dense":
                    add(L + "mlp.up", p[L + "up"][:fs["ff"]])
                    add(L + "mlp.down", p[L + "down"][:, :fs["ff"]])
                    act = p[L + "act"]
                    add(L + "mlp.act", act, "small",
                        put=lambda x, t=act, i=i: (t.copy_(x.reshape(t.shape)), self._act.pop(i, None)))
                else:
                    F = fs["ff"]
                    add(L + "mlp.router", p[L + "router"])
                    add(L + "mlp.router.b", p[L + "router.b"], "small")
                    for e in range(fs["experts"]):
                        add(L + f"mlp.e{e}.gate", p[L + "gate_up"][e, :F])
                        add(L + f"mlp.e{e}.up", p[L + "gate_up"][e, F:])
                        add(L + f"mlp.e{e}.down", p[L + "edown"][e])
        add("final.norm", p["final.norm"], "ones")
        add("final.norm.b", p["final.norm.b"], "small")
        return out

    @torch.no_grad()
    def init_random(self, seed: int = 0) -> None:
        """Deterministic random weights: each tensor is drawn on the host from a generator keyed on
        (seed, tensor name). Projections are scaled by 1 / sqrt(fan-in), the embedding so that the
        scaled rows have unit entries, norm weights sit around one, layer scales around 0.5, the
        depth average near 'mostly the newest layer'."""
        for lp in self.logical_params():
            g = torch.Generator().manual_seed(_name_seed(lp.name, seed))
            shp = lp.global_shape
            r = torch.randn(shp, generator=g)
            if lp.init == "normal":
                t = r / math.sqrt(shp[-1])
            elif lp.init == "embed":
                t = r / max(self.cfg.embed_scale, 1e-6)
            elif lp.init == "ones":
                t = 1.0 + 0.1 * r
            elif lp.init == "small":
                t = 0.1 * r
            elif lp.init == "scale":
                t = 0.5 + 0.1 * r
            elif lp.init == "taps":
                t = 0.3 * r
            elif lp.init == "avg":
                t = 0.1 * r
                t[-1] += 0.8
            else:
                raise ValueError(lp.init)
            # weights are bf16 values in every run (an f32 model holds them exactly)
            lp.set(t.to(torch.bfloat16).to(self.device))

    # ------------------------------------------------------------------------------------
    # caches
    # ------------------------------------------------------------------------------------
    def kv_bytes_per_token(self, dtype: Optional[torch.dtype] = None) -> int:
        es = torch.empty((), dtype=dtype or self.dtype).element_size()
        return max(1, sum(dk + dv for dk, dv in self.cache_dims) * es)

    def state_bytes_per_slot(self) -> int:
        return 4 * max(self.taps - 1, 0) * self.cfg.hidden_size * len(self.specs)

    def allocate_kv_cache(self, num_blocks: int, block_size: int, dtype: Optional[torch.dtype] = None) -> list:
        """Per layer one pair over the shared latent "head": K [blocks, 1, BS, kv_rank + rot_dim]
        rows [normed latent | rotated key part] and V [blocks, 1, kv_rank, BS], the latent again
        with a page's tokens contiguous (the P V operand)."""
        dt = dtype or self.dtype
        if dt != self.dtype:
            raise NotImplementedError("Zinesun caches hold the model's element type")
        return [(torch.zeros(num_blocks, 1, block_size, dk, dtype=dt, device=self.device),
                 torch.zeros(num_blocks, 1, dv, block_size, dtype=dt, device=self.device))
                for dk, dv in self.cache_dims]

    def allocate_state(self, num_slots: int) -> list:
        """The convolution history pool: one [slots, taps - 1, W] f32 tensor per layer (a sequence's
        last taps - 1 mixer inputs, oldest first)."""
        self.state = [torch.zeros(num_slots, self.taps - 1, self.cfg.hidden_size, dtype=torch.float32, device=self.device)
                      for _ in self.specs]
        return self.state

    # ------------------------------------------------------------------------------------
    # forward
    # ------------------------------------------------------------------------------------
    def _act_coeffs(self, i: int, pre: str) -> tuple:
        """xIELU coefficients of layer i: (softplus(p), 1/2 + softplus(q)) from the stored pair."""
        a = self._act.get(i)
        if a is None:
            v = self.p[pre + "act"].tolist()
            a = self._act[i] = (_softplus(v[0]), 0.5 + _softplus(v[1]))
        return a

    def prepare(self) -> None:
        """Host-side constants derived from weights (read once, outside any graph capture)."""
        for sp in self.specs:
            if sp["ffn"] and sp["ffn"]["kind"] == "dense":
                self._act_coeffs(sp["index"], f"l{sp['index']}.")

    def forward(self, fb: ForwardBatch, kv_caches: Optional[list] = None,
                hidden_in: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One step over the packed rows of `fb`; returns f32 logits [R, padded vocab] for the rows
        fb.logits_idx names (None: all)."""
        p, c, eps = self.p, self.cfg, self.cfg.norm_eps
        meta = self._step_meta(fb)
        T, W, L = fb.num_tokens, c.hidden_size, len(self.specs)
        if self.has_state and T and not self.state:
            raise RuntimeError("Zinesun: the convolution history pool is not allocated (KVCache state slots)")
        # results of the embedding and of every layer (the depth average reads all of them)
        stack = ops.new_empty(L + 1, T, W, dtype=torch.float32, device=self.device)
        ops.embed_scaled(fb.input_ids, p["embed"], c.embed_scale, out=stack[0])
        x = stack[0]
        xbuf = ops.new_empty(T, W, dtype=torch.float32, device=self.device)
        for n, sp in enumerate(self.specs):
            pre = f"l{sp['index']}."
            st = self.state[n] if self.has_state else None
            h = ops.conv_mix(x, p.get(pre + "canon1"), st, meta["state_slots"], meta["row_cu"], fb.positions, self.dtype)
            if st is not None:
                ops.conv_state_update_(x, st, meta["state_slots"], meta["row_cu"], fb.positions)
            y = self._latent_attention(sp, pre, h, fb, meta, kv_caches)
            fs = sp["ffn"]
            hx = ops.post_norm_add(x, y, p[pre + "norm1"], p[pre + "norm1.b"], eps, p[pre + "ls1"], out=xbuf,
                                   cast_dtype=self.dtype if fs else None)
            f = self._ffn(sp, pre, hx) if fs else None
            ops.post_norm_add_avg(xbuf, f, p.get(pre + "norm2"), p.get(pre + "norm2.b"), eps, p.get(pre + "ls2"),
                                  stack, n + 1, p[pre + "dwa"])
            x = xbuf
            if self.layer_probe is not None:
                self.layer_probe(sp["index"], x)
        xf = ops.layer_norm_rows(x, p["final.norm"], p["final.norm.b"], eps, fb.logits_idx, self.dtype)
        return ops.linear_act(xf, p["embed"], out_dtype=torch.float32)

    def _latent_attention(self, sp, pre, h, fb, meta, kv_caches):
        T = fb.num_tokens
        H, D, Dv, R, Q, rd = sp["heads"], sp["dim"], sp["vdim"], sp["kv_rank"], sp["q_rank"], sp["rot_dim"]
        if kv_caches is None:
            raise RuntimeError("Zinesun attention runs through the paged cache")
        kc, vc = kv_caches[self.cache_index[sp["index"]]]
        p = self.p
        z = ops.linear_act(h, p[pre + "in"])
        cq, gate = ops.latent_prep(z, Q, R, rd, H, p[pre + "dq.norm"], p[pre + "dkv.norm"], self.cfg.norm_eps,
                                   fb.positions, p[pre + "inv_freq"], fb.slots, kc, vc, self.dtype)
        q = ops.linear_act(cq, p[pre + "uq"])[:, :H * (D + rd)].view(T, H, D + rd)
        # queries in the latent space: [W_uk^T q_nope | rotated q_rot] per head
        ql = ops.new_empty(T, H, kc.shape[3], dtype=self.dtype, device=self.device)
        ops.linear_heads(q[:, :, :D], p[pre + "ukT"], ql[:, :, :R])
        ops.rope_heads_copy(q[:, :, D:], ql[:, :, R:], fb.positions, p[pre + "inv_freq"])    # (zero-fills the padding)
        ol = ops.attn_window_paged(ql, kc, vc, meta["tables"], meta["row_cu"], fb.positions, sp["scale"], sp["window"],
                                   0, None, row_map=meta["row_map"], fold_heads=True, out_scale=gate)
        o = ops.new_empty(T, H, Dv, dtype=self.dtype, device=self.device)
        ops.linear_heads(ol[:, :, :R], p[pre + "uv"], o)
        return ops.linear_act(o.view(T, H * Dv), p[pre + "o"])

    def _ffn(self, sp, pre, h):
        fs, p = sp["ffn"], self.p
        if fs["kind"] == "dense":
            a = ops.linear_act(h, p[pre + "up"], act="xielu", act_params=self._act_coeffs(sp["index"], pre))
            return ops.linear_act(a, p[pre + "down"])
        ids, w = ops.moe_route_scores(h, p[pre + "router"], fs["top"], scoring="softmax", renorm=True,
                                      bias=p[pre + "router.b"])
        return ops.moe_glu_ffn(h, ids, w, p[pre + "gate_up"], p[pre + "edown"], float("inf"), 1.0, up_offset=0.0,
                               scale_input=False)
