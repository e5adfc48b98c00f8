"""Nesizen: a decoder-only LM whose layers differ from one another (ModelConfig.layer_specs).

  embedding   : token rows, RMS norm with a weight stored around zero (x / rms * (1 + w)), copied
                into `residual_streams` parallel f32 residual streams (hyper-connections)
  every layer : for the mixer and, if the layer has one, the feed-forward:
                  h = norm(sum_s in[s] x_s);  y = sublayer(h);
                  x_r <- sum_s mix[s, r] x_s + out[r] y      (all streams from the old ones)
    mixer "attention" : GQA with per-layer head sizes (value size may differ from the key size),
                        interleaved-pair rotary on the first rot_dims dims, a causal sliding
                        window that also keeps the first keep_first positions, a learned per-head
                        sink logit in the softmax denominator; a layer may read the keys / values
                        another layer cached (kv_from) with its own queries
    mixer "gla"       : gated linear attention, S <- diag(a) S + k v^T, o = S^T q, with a
                        low-rank data-dependent decay a = sigmoid(W2 W1 h + b)^(1/tau), per-head
                        RMS norm of o, a silu gate; the state lives in the cache's per-sequence
                        state slots (f32)
    feed-forward      : dense squared-ReLU MLP, or sigmoid-scored top-k MoE whose experts are
                        clamped GLUs run on (score * h), scores not renormalised
  output      : sum of the streams, the offset-weight norm, LM head

Every size and constant comes from the config; residual streams, norms, softmax, rotary angles,
decays, recurrent state and router run in f32 in the bf16 model too. The model runs unsharded
(tp = pp = ep = 1; data-parallel replicas are independent engines). Prompt chunks always attend
through the paged cache (`paged_prefill_only`), so one attention kernel serves fresh prompts,
continuation chunks and decoded tokens and a position's result does not depend on how the
prompt was cut.
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
from .stack import PackedStack, pad128 as _pad128
from .transformer import LogicalParam, _name_seed


NORM_OFFSET = 1.0       # norm weights are stored around zero
GLU_ALPHA = 1.702       # expert activation g * sigmoid(alpha g)


class NesizenLM(PackedStack):
    def __init__(self, cfg: ModelConfig, shard: Shard = Shard(), device="cpu",
                 dtype: torch.dtype = torch.bfloat16, comm: Optional[Communicator] = None):
        if not cfg.layer_specs:
            raise ValueError("Nesizen needs ModelConfig.layer_specs (ModelConfig.from_nesizen)")
        if shard.tp_size != 1 or shard.ep_size != 1 or shard.layer_start != 0 or \
                (shard.layer_end is not None and shard.layer_end != cfg.num_layers):
            raise NotImplementedError("Nesizen runs unsharded (tp = pp = ep = 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Nesizen runs in bfloat16 or float32")
        self.cfg, self.shard = cfg, shard
        self.device, self.dtype = torch.device(device), dtype
        self.comm = comm or Communicator.single()
        self.specs = cfg.layer_specs
        self.streams = cfg.residual_streams
        self.layer_ids = list(range(cfg.num_layers))
        self.first = self.last = True
        self.tp = self.ep = 1
        vpad = (cfg.vocab_size + 127) // 128 * 128
        self.dims = LocalDims(hq=cfg.num_heads, hkv=cfg.num_kv_heads, kv_head0=0, q_head0=0,
                              ffn=max(cfg.intermediate_size, 1), ffn0=0, vocab=vpad, vocab0=0, vocab_padded=vpad,
                              experts=max(cfg.num_experts, 1), expert0=0)
        # paged caches exist for attention layers with their own keys; sharing layers point at them
        self.cache_index: dict[int, int] = {}
        for sp in self.specs:
            if sp["type"] == "attention" and sp["kv_from"] is None:
                self.cache_index[sp["index"]] = len(self.cache_index)
        for sp in self.specs:
            if sp["type"] == "attention" and sp["kv_from"] is not None:
                self.cache_index[sp["index"]] = self.cache_index[sp["kv_from"]]
        self.state_index = {sp["index"]: n for n, sp in
                            enumerate(s for s in self.specs if s["type"] == "gla")}
        self.has_state = bool(self.state_index)
        self.state: list = []             # set by allocate_state (the cache object owns the pool)
        self.layer_probe = None           # debug hook: f(layer, residual [T, W] f32) after every layer
        self.p: dict[str, torch.Tensor] = {}
        self.packed: dict = {}
        self._arange: dict = {}
        self._alloc()

    # ------------------------------------------------------------------------------------
    # parameters
    # ------------------------------------------------------------------------------------
    def _alloc(self):
        c, W = self.cfg, self.cfg.hidden_size
        z = lambda *s: torch.zeros(*s, dtype=self.dtype, device=self.device)                  # noqa: E731
        f = lambda *s: torch.zeros(*s, dtype=torch.float32, device=self.device)               # noqa: E731
        p = self.p
        p["embed"], p["embed.norm"] = z(c.vocab_size, W), f(W)
        S = self.streams
        for sp in self.specs:
            pre = f"l{sp['index']}."
            H, D, Dv = sp["heads"], sp["dim"], sp["vdim"]
            p[pre + "norm1"] = f(W)
            p[pre + "hc1.in"], p[pre + "hc1.out"], p[pre + "hc1.mix"] = f(S), f(S), f(S, S)
            if sp["type"] == "attention":
                G = sp["kv_heads"]
                own = sp["kv_from"] is None
                p[pre + "qkv"] = z(_pad128(H * D + (G * (D + Dv) if own else 0)), W)
                p[pre + "sink"] = f(H)
                n = sp["rot_dims"] // 2
                i = torch.arange(n, dtype=torch.float64)
                p[pre + "inv_freq"] = (sp["rot_base"] ** (-2.0 * i / max(sp["rot_dims"], 1))).to(torch.float32).to(self.device)
            else:
                # the fused projection and a2 are sized by _size_gla (they depend on the decay rank)
                p[pre + "a2b"], p[pre + "gnorm"] = z(H * D), f(Dv)
            p[pre + "o"] = z(W, H * Dv)
            fs = sp["ffn"]
            if fs:
                p[pre + "norm2"] = f(W)
                p[pre + "hc2.in"], p[pre + "hc2.out"], p[pre + "hc2.mix"] = f(S), f(S), f(S, S)
                if fs["kind"] == "dense":
                    p[pre + "up"], p[pre + "down"] = z(fs["ff"], W), z(W, fs["ff"])
                else:
                    E, F = fs["experts"], fs["ff"]
                    p[pre + "router"] = z(E, W)
                    p[pre + "gate_up"], p[pre + "edown"] = z(E, 2 * F, W), z(E, W, F)
        p["final.norm"] = f(W)
        p["head"] = z(self.dims.vocab, W)
        for sp in self.specs:
            if sp["type"] == "gla":
                self._size_gla(sp, sp.get("decay_rank") or 16)

    def _size_gla(self, sp: dict, rank: int) -> None:
        """(Re)allocate the fused projection of a GLA layer for decay rank `rank`: rows
        q | k | v | gate | a1. The rank is a tensor shape (a1 [rank, W]), known from the checkpoint
        or chosen by the random initialiser."""
        W, H, D, Dv = self.cfg.hidden_size, sp["heads"], sp["dim"], sp["vdim"]
        pre = f"l{sp['index']}."
        sp["decay_rank"] = int(rank)
        self.p[pre + "qkvga"] = torch.zeros(_pad128(2 * H * D + 2 * H * Dv + rank), W, dtype=self.dtype, device=self.device)
        self.p[pre + "a2"] = torch.zeros(H * D, rank, dtype=self.dtype, device=self.device)

    def set_decay_ranks(self, shapes: dict) -> None:
        """Take each GLA layer's decay rank from checkpoint tensor shapes {name: shape}."""
        for sp in self.specs:
            if sp["type"] == "gla":
                shp = shapes.get(f"l{sp['index']}.mix.a1")
                if shp is not None and int(shp[0]) != sp["decay_rank"]:
                    self._size_gla(sp, int(shp[0]))

    @property
    def head_weight(self) -> torch.Tensor:
        return self.p["head"]

    def logical_params(self) -> list[LogicalParam]:
        """Checkpoint tensors by their file names ('l<i>.mix.q', 'l<i>.mlp.e<j>.gate', ...), each
        a view into the fused local tensors."""
        c, p = self.cfg, self.p
        out: list[LogicalParam] = []

        def add(name, t, init="normal"):
            out.append(LogicalParam(name, tuple(t.shape), None, 0, 0, init, (lambda t=t: t),
                                    (lambda x, t=t: t.copy_(x.reshape(t.shape)))))

        add("embed", p["embed"])
        add("embed.norm", p["embed.norm"], "norm")
        for sp in self.specs:
            i = sp["index"]
            pre, L = f"l{i}.", f"l{i}."
            H, D, Dv = sp["heads"], sp["dim"], sp["vdim"]
            add(L + "norm1", p[pre + "norm1"], "norm")
            for q in ("1", "2") if sp["ffn"] else ("1",):
                add(L + f"hc{q}.in", p[pre + f"hc{q}.in"], "hc_in")
                add(L + f"hc{q}.out", p[pre + f"hc{q}.out"], "hc_out")
                add(L + f"hc{q}.mix", p[pre + f"hc{q}.mix"], "hc_mix")
            if sp["type"] == "attention":
                qkv, G = p[pre + "qkv"], sp["kv_heads"]
                add(L + "mix.q", qkv[:H * D])
                if sp["kv_from"] is None:
                    add(L + "mix.k", qkv[H * D:H * D + G * D])
                    add(L + "mix.v", qkv[H * D + G * D:H * D + G * D + G * sp["vdim"]])
                add(L + "mix.sink", p[pre + "sink"], "sink")
            else:
                fz, r = p[pre + "qkvga"], sp["decay_rank"]
                o1, o2, o3, o4 = H * D, 2 * H * D, 2 * H * D + H * Dv, 2 * H * D + 2 * H * Dv
                add(L + "mix.q", fz[:o1])
                add(L + "mix.k", fz[o1:o2])
                add(L + "mix.v", fz[o2:o3])
                add(L + "mix.g", fz[o3:o4])
                add(L + "mix.a1", fz[o4:o4 + r])
                add(L + "mix.a2", p[pre + "a2"])
                add(L + "mix.a2.b", p[pre + "a2b"], "decay_bias")
                add(L + "mix.norm", p[pre + "gnorm"], "ones")
            add(L + "mix.o", p[pre + "o"])
            fs = sp["ffn"]
            if fs:
                add(L + "norm2", p[pre + "norm2"], "norm")
                if fs["kind"] == "dense":
                    add(L + "mlp.up", p[pre + "up"])
                    add(L + "mlp.down", p[pre + "down"])
                else:
                    F = fs["ff"]
                    add(L + "mlp.router", p[pre + "router"])
                    for e in range(fs["experts"]):
                        add(L + f"mlp.e{e}.gate", p[pre + "gate_up"][e, :F])
                        add(L + f"mlp.e{e}.up", p[pre + "gate_up"][e, F:])
                        add(L + f"mlp.e{e}.down", p[pre + "edown"][e])
        add("final.norm", p["final.norm"], "norm")
        add("head", p["head"][:c.vocab_size])
        return out

    @torch.no_grad()
    def init_random(self, seed: int = 0) -> None:
        """Deterministic random weights: each tensor is drawn on the host from a generator keyed
        on (seed, tensor name). Projections are scaled by 1 / sqrt(fan-in); norm weights sit
        around zero, stream mixers around the identity, decay biases so that decays are near 1."""
        S = self.streams
        for lp in self.logical_params():
            g = torch.Generator().manual_seed(_name_seed(lp.name, seed))
            shp = lp.global_shape
            r = torch.randn(shp, generator=g)
            if lp.init == "normal":
                t = r / math.sqrt(shp[-1]) if len(shp) > 1 else r
            elif lp.init == "norm":
                t = 0.1 * r
            elif lp.init == "ones":
                t = 1.0 + 0.1 * r
            elif lp.init == "hc_in":
                t = 1.0 / S + 0.1 * r
            elif lp.init == "hc_out":
                t = 1.0 + 0.1 * r
            elif lp.init == "hc_mix":
                t = torch.eye(S) + 0.1 * r
            elif lp.init == "sink":
                t = r
            elif lp.init == "decay_bias":
                t = 2.0 + r
            else:
                raise ValueError(lp.init)
            # weights are bf16 values in every run (an f32 model holds them exactly)
            lp.set(t.to(torch.bfloat16).to(self.device))

    # ------------------------------------------------------------------------------------
    # caches
    # ------------------------------------------------------------------------------------
    def state_bytes_per_slot(self) -> int:
        return sum(4 * sp["heads"] * sp["dim"] * sp["vdim"] for sp in self.specs if sp["type"] == "gla")

    def allocate_kv_cache(self, num_blocks: int, block_size: int, dtype: Optional[torch.dtype] = None) -> list:
        """One (K [blocks, G, BS, D], V [blocks, G, Dv, BS]) pair per attention layer that has its
        own keys, in layer order (`cache_index` maps a layer to its pair)."""
        dt = dtype or self.dtype
        if dt != self.dtype:
            raise NotImplementedError("Nesizen caches hold the model's element type")
        caches = []
        for sp in self.specs:
            if sp["type"] == "attention" and sp["kv_from"] is None:
                G = sp["kv_heads"]
                caches.append((torch.zeros(num_blocks, G, block_size, sp["dim"], dtype=dt, device=self.device),
                               torch.zeros(num_blocks, G, sp["vdim"], block_size, dtype=dt, device=self.device)))
        return caches

    def allocate_state(self, num_slots: int) -> list:
        """The recurrent-state pool: one [slots, H, D, Dv] f32 tensor per GLA layer."""
        self.state = [torch.zeros(num_slots, sp["heads"], sp["dim"], sp["vdim"], dtype=torch.float32, device=self.device)
                      for sp in self.specs if sp["type"] == "gla"]
        return self.state

    # ------------------------------------------------------------------------------------
    # forward
    # ------------------------------------------------------------------------------------
    def forward(self, fb: ForwardBatch, kv_caches: Optional[list] = None,
                hidden_in: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One step over the packed rows of `fb`; returns logits [R, padded vocab] for the rows
        fb.logits_idx names (None: all)."""
        p, eps = self.p, self.cfg.norm_eps
        meta = self._step_meta(fb)
        xs = ops.embed_norm_streams(fb.input_ids, p["embed"], p["embed.norm"], eps, NORM_OFFSET, self.streams)
        # sublayers in order; each stream update is fused with the next sublayer's mixed-in norm
        subs = [(sp, q) for sp in self.specs for q in ((1, 2) if sp["ffn"] else (1,))]
        sp0 = subs[0][0]
        h = ops.hc_pre(xs, p[f"l{sp0['index']}.hc1.in"], p[f"l{sp0['index']}.norm1"], eps, NORM_OFFSET, self.dtype)
        for n, (sp, q) in enumerate(subs):
            pre = f"l{sp['index']}."
            if q == 2:
                y = self._ffn(sp["ffn"], pre, h)
            elif sp["type"] == "attention":
                y = self._attention(sp, pre, h, fb, meta, kv_caches)
            else:
                y = self._gla(sp, pre, h, fb, meta)
            hc = pre + f"hc{q}."
            if n + 1 < len(subs):
                nsp, nq = subs[n + 1]
                npre = f"l{nsp['index']}."
                h = ops.hc_post_pre_(xs, y, p[hc + "mix"], p[hc + "out"], p[npre + f"hc{nq}.in"], p[npre + f"norm{nq}"],
                                     eps, NORM_OFFSET, self.dtype)
            else:
                ops.hc_post_(xs, y, p[hc + "mix"], p[hc + "out"])
            if self.layer_probe is not None and (q == 2 or not sp["ffn"]):
                self.layer_probe(sp["index"], xs.sum(1))
        x = ops.hc_final(xs, p["final.norm"], eps, NORM_OFFSET, fb.logits_idx, self.dtype)
        return ops.linear_act(x, p["head"])

    def _attention(self, sp, pre, h, fb, meta, kv_caches):
        T = fb.num_tokens
        H, G, D, Dv = sp["heads"], sp["kv_heads"], sp["dim"], sp["vdim"]
        if kv_caches is None:
            raise RuntimeError("Nesizen attention runs through the paged cache")
        kc, vc = kv_caches[self.cache_index[sp["index"]]]
        qkv = ops.linear_act(h, self.p[pre + "qkv"])
        q = qkv[:, :H * D].view(T, H, D)
        if sp["kv_from"] is None:
            k = qkv[:, H * D:H * D + G * D].view(T, G, D)
            v = qkv[:, H * D + G * D:H * D + G * (D + Dv)].view(T, G, Dv)
            ops.rope_partial_kv(q, k, v, fb.positions, self.p[pre + "inv_freq"], fb.slots, kc, vc)
        else:
            ops.rope_partial_kv(q, None, None, fb.positions, self.p[pre + "inv_freq"])
        o = ops.attn_window_paged(q, kc, vc, meta["tables"], meta["row_cu"], fb.positions, sp["scale"], sp["window"],
                                  sp["keep_first"], self.p[pre + "sink"], row_map=meta["row_map"])
        return ops.linear_act(o.view(T, H * Dv), self.p[pre + "o"])

    def _gla(self, sp, pre, h, fb, meta):
        T = fb.num_tokens
        H, D, Dv, r = sp["heads"], sp["dim"], sp["vdim"], sp["decay_rank"]
        fz = ops.linear_act(h, self.p[pre + "qkvga"])
        o1, o2, o3, o4 = H * D, 2 * H * D, 2 * H * D + H * Dv, 2 * H * D + 2 * H * Dv
        q, k = fz[:, :o1].view(T, H, D), fz[:, o1:o2].view(T, H, D)
        v, g = fz[:, o2:o3].view(T, H, Dv), fz[:, o3:o4]
        z = ops.linear_act(fz[:, o4:o4 + r], self.p[pre + "a2"], bias=self.p[pre + "a2b"])
        o = ops.gla_scan(q, k, v, z, self.state[self.state_index[sp["index"]]], meta["state_slots"], meta["row_cu"],
                         fb.positions, sp["tau"], D ** -0.5)
        y = ops.gla_out(o, g, self.p[pre + "gnorm"], self.cfg.norm_eps, self.dtype)
        return ops.linear_act(y, self.p[pre + "o"])

    def _ffn(self, fs, pre, h):
        if fs["kind"] == "dense":
            return ops.linear_act(ops.linear_act(h, self.p[pre + "up"], act="relu2"), self.p[pre + "down"])
        ids, w = ops.moe_route_scores(h, self.p[pre + "router"], fs["top"], scoring="sigmoid", renorm=False)
        return ops.moe_glu_ffn(h, ids, w, self.p[pre + "gate_up"], self.p[pre + "edown"],
                               float("inf") if fs["limit"] is None else fs["limit"], GLU_ALPHA)
