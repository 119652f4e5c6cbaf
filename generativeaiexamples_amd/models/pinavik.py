"""Pinavik: a hybrid decoder whose layer list mixes three token mixers, with a looped block of layers.

Architecture (every size and constant comes from ``config.json``; the layer list may hold the mixers in any order):
  * embedding times ``embedding.scale``; pre-norm layers ``x += m * mixer(norm1(x)); x += m * ff(norm2(x))`` with
    ``m = residual_mult`` and zero-centred RMS-norm weights (``x / rms(x) * (1 + w)``); a layer may have no
    feed-forward;
  * ``loop``: layers ``start .. stop-1`` run ``times`` times with the same weights (each pass with its own KV cache /
    recurrent state). Before every pass ``x <- W_in [x ; x0] + step[pass]`` with ``x0`` the embedding output;
  * mixer ``attention``: GQA without rotation; q and k are RMS-normalised over their WHOLE projection (all heads at
    once); scores ``scale * q.k`` pass ``cap * tanh(. / cap)`` and lose ``r1_h ln(1 + r2_h (i - j))``; sliding
    window ``0 <= i - j < mask.size``; heads times ``sigmoid(W_g h)`` before the output projection;
  * mixer ``wkv``: token-shift mixes ``h + (h_prev - h) mu_s`` for r, k, v, g, w; per-channel decay
    ``exp(-exp(W_w2 tanh(W_w1 m_w) + w0))``; state ``S <- diag(w) S + k v^T`` read as ``(S + diag(u) k v^T)^T r``;
    per-head RMS norm, weight, ``silu`` gate, output projection;
  * mixer ``channel_delta``: gated delta rule with one decay per head and key channel; q, k, v pass a short causal
    depthwise convolution + SiLU; unit-norm q (times ``dim^-1/2``) and k; ``beta = sigmoid(W_b h)``; low-rank decay
    and output-gate projections; per-head RMS norm with a shared weight, ``sigmoid`` gate, output projection;
  * feed-forward ``W_down polynorm(W_up h)`` with ``polynorm(z) = a N(z) + b N(z^2) + c N(z^3) + e``;
  * final zero-centred RMS norm and the output head.

MI355X mapping: the residual stream, every norm statistic, attention scores / softmax, decays and the recurrent
states are fp32; the projections run in the model dtype (bf16 on the MFMA GEMMs with fp32 accumulation, or true fp32).
Attention runs keep K / V in the engine's paged cache (one cache layer per attention layer RUN, each with its own head
geometry); the recurrent runs keep their fp32 states (token-shift row, conv window, S matrices) in the engine's state
slot pool. A step's rows - prompt portions and single decoded tokens alike - go through the same HIP kernels
(``ops.window_attention``, ``ops.wkv_scan``, ``ops.delta_scan`` ...), addressed by device-side (cu, slot, ctx) vectors,
so pure-decode steps replay a captured HIP graph. The q|k|v|gate projections of an attention layer and the
q|k|v|a1|g1|b projections of a delta layer are fused into one GEMM each at load time; every residual add is fused with
the following RMS norm.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from .. import ops
from ..engine.state_pool import StatePool
from ..parallel.dist import DistContext, get_context
from .common import ForwardBatch

MIXERS = ("attention", "wkv", "channel_delta")


@dataclass
class PinavikConfig:
    vocab_size: int
    hidden_size: int
    layers: Tuple[dict, ...]                 # {"type", "mixer": {...}, "mlp": {"kind", "ff"} | None}
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0                      # 0: no looped block
    rms_eps: float = 1e-6
    residual_mult: float = 1.0
    embedding_scale: float = 1.0
    name: str = "pinavik"
    max_position: int = 1 << 20              # positions enter only through distances: no table to outgrow
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()

    def __post_init__(self):
        layers = []
        for i, l in enumerate(self.layers):
            if l["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
            if l.get("mlp") is not None and l["mlp"].get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {l['mlp'].get('kind')!r}")
            m = dict(l["mixer"])  # optional keys get their neutral values: MHA, values as wide as keys, 1 / sqrt(dim)
            if l["type"] != "wkv":
                m.setdefault("kv_heads", m["heads"])
                m.setdefault("vdim", m["dim"])
                if m["heads"] % m["kv_heads"]:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            if l["type"] == "attention":
                m.setdefault("scale", m["dim"] ** -0.5)
            layers.append(dict(l, mixer=m, mlp=l.get("mlp")))
        self.layers = tuple(layers)
        if self.loop_times and not (0 <= self.loop_start < self.loop_stop <= len(self.layers)):
            raise ValueError("loop: need 0 <= start < stop <= number of layers")

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def head_dim(self) -> int:  # engine sizing hooks: the widest attention head
        return max([l["mixer"]["dim"] for l in self.layers if l["type"] == "attention"] or [16])

    def runs(self) -> List[Tuple[int, int]]:
        """Execution order as (layer, pass) pairs; a looped layer appears once per pass."""
        n = len(self.layers)
        if not self.loop_times:
            return [(i, 0) for i in range(n)]
        out = [(i, 0) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            out += [(i, t) for i in range(self.loop_start, self.loop_stop)]
        return out + [(i, 0) for i in range(self.loop_stop, n)]

    @staticmethod
    def from_json(path_or_dict) -> "PinavikConfig":
        if isinstance(path_or_dict, dict):
            c, name = path_or_dict, "pinavik"
        else:
            with open(os.path.join(path_or_dict, "config.json")) as f:
                c = json.load(f)
            name = os.path.basename(os.path.normpath(path_or_dict)) or "pinavik"
        lp = c.get("loop") or {}
        eos = c.get("eos_token_id", ())
        return PinavikConfig(
            vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(c["layers"]),
            loop_start=int(lp.get("start", 0)), loop_stop=int(lp.get("stop", 0)), loop_times=int(lp.get("times", 0)),
            rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)), residual_mult=float(c.get("residual_mult", 1.0)),
            embedding_scale=float((c.get("embedding") or {}).get("scale", 1.0)), name=c.get("name", name),
            max_position=int(c.get("max_position", 1 << 20)), bos_token_id=c.get("bos_token_id"),
            eos_token_ids=tuple(eos) if isinstance(eos, (list, tuple)) else (eos,))

    @staticmethod
    def tiny(**kw) -> "PinavikConfig":
        att = dict(dim=32, vdim=16, heads=4, kv_heads=2, mask=dict(size=24), scale=0.2, softcap=20.0)
        wkv = dict(dim=16, heads=4)
        cd = dict(dim=16, vdim=32, heads=4, kv_heads=2, conv=3)
        mlp = dict(kind="dense", ff=128)
        base = dict(vocab_size=512, hidden_size=64, name="tiny-pinavik", rms_eps=1e-5, residual_mult=0.5,
                    embedding_scale=8.0, loop_start=1, loop_stop=3, loop_times=2,
                    layers=(dict(type="wkv", mixer=wkv, mlp=mlp), dict(type="attention", mixer=att, mlp=mlp),
                            dict(type="channel_delta", mixer=cd, mlp=None), dict(type="attention", mixer=att, mlp=mlp)))
        base.update(kw)
        return PinavikConfig(**base)

    @staticmethod
    def sized(width: int, n_layers: int, ff: int, heads: int, head_dim: int, window: int = 1024, vocab: int = 32768,
              pattern: Tuple[str, ...] = MIXERS, **kw) -> "PinavikConfig":
        """A regular stack for benchmarks: `pattern` repeated over n_layers, equal head geometry in every mixer."""
        mix = dict(attention=dict(dim=head_dim, vdim=head_dim, heads=heads, kv_heads=max(1, heads // 4),
                                  mask=dict(size=window), scale=head_dim ** -0.5, softcap=30.0),
                   wkv=dict(dim=head_dim, heads=heads),
                   channel_delta=dict(dim=head_dim, vdim=head_dim, heads=heads, kv_heads=max(1, heads // 2), conv=4))
        layers = tuple(dict(type=pattern[i % len(pattern)], mixer=mix[pattern[i % len(pattern)]],
                            mlp=dict(kind="dense", ff=ff)) for i in range(n_layers))
        base = dict(vocab_size=vocab, hidden_size=width, layers=layers, embedding_scale=math.sqrt(width),
                    residual_mult=0.5, name=f"pinavik-{width}x{n_layers}")
        base.update(kw)
        return PinavikConfig(**base)


def random_state(cfg: PinavikConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """A random checkpoint (tensor names and shapes of the safetensors layout, fp32 values) with magnitudes that keep
    activations, decays and states in a trained model's range."""
    g = torch.Generator().manual_seed(seed)
    D = cfg.hidden_size
    rn = lambda *s, std=1.0: torch.randn(*s, generator=g) * std  # noqa: E731
    un = lambda *s, lo=0.0, hi=1.0: torch.rand(*s, generator=g) * (hi - lo) + lo  # noqa: E731
    lin = lambda o, i: rn(o, i, std=i ** -0.5)  # noqa: E731
    sd: Dict[str, torch.Tensor] = {"embed": rn(cfg.vocab_size, D, std=1.0 / max(cfg.embedding_scale, 1e-3)),
                                   "head": lin(cfg.vocab_size, D), "final.norm": rn(D, std=0.1)}
    if cfg.loop_times:
        sd["loop.in"] = lin(D, 2 * D) * math.sqrt(2.0)
        sd["loop.step"] = rn(cfg.loop_times, D, std=0.1)
    for i, l in enumerate(cfg.layers):
        p, m = f"l{i}.", l["mixer"]
        sd[p + "norm1"] = rn(D, std=0.1)
        x = p + "mix."
        if l["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            sd[x + "q"], sd[x + "k"], sd[x + "v"] = lin(H * dk, D), lin(G * dk, D), lin(G * dv, D)
            sd[x + "q.norm"], sd[x + "k.norm"] = 1 + rn(H * dk, std=0.1), 1 + rn(G * dk, std=0.1)
            sd[x + "r1"], sd[x + "r2"] = un(H, lo=0.1, hi=1.0), un(H, lo=0.05, hi=1.0)
            sd[x + "g"], sd[x + "o"] = lin(H * dv, D), lin(D, H * dv)
        elif l["type"] == "wkv":
            H, d = m["heads"], m["dim"]
            r = max(8, D // 16)
            for s_ in "rkvgw":
                sd[x + "mu." + s_] = un(D)
            for s_ in "rkvg":
                sd[x + s_] = lin(H * d, D)
            sd[x + "k"] = sd[x + "k"] * d ** -0.5
            sd[x + "w1"], sd[x + "w2"] = lin(r, D), lin(H * d, r)
            sd[x + "w0"] = un(H * d, lo=-4.0, hi=0.5)
            sd[x + "u"] = rn(H, d, std=0.3)
            sd[x + "norm"] = 1 + rn(H * d, std=0.1)
            sd[x + "o"] = lin(D, H * d)
        else:
            H, G, dk, dv, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            r = max(8, D // 16)
            for s_, n in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
                sd[x + s_] = lin(n, D)
                sd[x + s_ + ".conv"] = rn(n, K, std=K ** -0.5)
            sd[x + "b"] = lin(H, D)
            sd[x + "A_log"] = torch.log(un(H, lo=0.5, hi=4.0))
            sd[x + "norm"] = 1 + rn(dv, std=0.1)
            sd[x + "a1"], sd[x + "a2"] = lin(r, D), lin(H * dk, r)
            sd[x + "dt_bias"] = un(H * dk, lo=-4.0, hi=0.0)
            sd[x + "g1"], sd[x + "g2"] = lin(r, D), lin(H * dv, r)
            sd[x + "o"] = lin(D, H * dv)
        if l.get("mlp") is not None:
            F_ = l["mlp"]["ff"]
            sd[p + "norm2"] = rn(D, std=0.1)
            sd[p + "mlp.up"], sd[p + "mlp.down"] = lin(F_, D), lin(D, F_)
            sd[p + "mlp.act"] = torch.tensor([0.6, 0.3, 0.2, 0.05]) + rn(4, std=0.05)
    return sd


class PinavikModel:
    """Weights (plain tensors) + forward for the serving engine (the hooks of LlamaModel / Qwen3NextModel)."""

    has_recurrent_state = True       # no prefix-cache reuse: a cached prefix has no recurrent state to resume from
    attention_backend = "window"     # ops.window_attention: no flash-attention tile lists / split-key workspace

    def __init__(self, cfg: PinavikConfig, device=None, dtype=torch.bfloat16, dist_ctx: DistContext | None = None,
                 state_slots: Optional[int] = None):
        self.cfg = cfg
        self.ctx = dist_ctx or get_context()
        assert self.ctx.tp_size == 1, "Pinavik runs TP=1"
        self.device = torch.device(device) if device is not None else self.ctx.device
        self.dtype = dtype
        self.runs = cfg.runs()
        att = [r for r in self.runs if cfg.layers[r[0]]["type"] == "attention"]
        self.kv_index = {r: j for j, r in enumerate(att)}
        self.num_kv_layers = len(att)
        heads = [cfg.layers[i]["mixer"] for i, _ in att]
        self.hq = max([m["heads"] for m in heads] or [1])
        self.hkv = max([m["kv_heads"] for m in heads] or [1])
        self.vocab_local, self.vstart = cfg.vocab_size, 0
        self.lora_names: list = []
        self.w: Dict[str, torch.Tensor] = {}
        self.pool = StatePool(state_slots or int(os.environ.get("GAI_LINEAR_STATE_SLOTS", "64")), self.device)
        self.state: Dict[Tuple[int, int], Dict[str, torch.Tensor]] = {}
        self.capture_residuals: Optional[list] = None  # numerics debugging: the residual stream after every layer run
        self._i32 = dict(dtype=torch.int32, device=self.device)

    # ------------------------------------------------------------------ engine sizing hooks
    def kv_layout(self) -> List[Tuple[int, int, int]]:
        """(kv heads, key size, value size) of every paged cache layer: one per attention layer run."""
        out = []
        for (i, _t) in sorted(self.kv_index, key=self.kv_index.get):
            m = self.cfg.layers[i]["mixer"]
            out.append((m["kv_heads"], m["dim"], m["vdim"]))
        return out

    # ------------------------------------------------------------------ weights
    def load_state(self, sd: Dict[str, torch.Tensor]):
        """Checkpoint tensors (the safetensors names) -> device weights: projections in the model dtype, per-channel
        tables fp32, zero-centred norm weights folded to 1 + w, same-input projections fused."""
        c, dev, dt = self.cfg, self.device, self.dtype
        f32 = lambda t: t.to(torch.float32).to(dev).contiguous()  # noqa: E731
        mat = lambda t: t.to(torch.float32).to(dev, dt).contiguous()  # noqa: E731
        w = self.w = {}
        w["embed"], w["head"] = mat(sd["embed"]), mat(sd["head"])
        w["final.norm"] = 1.0 + f32(sd["final.norm"])
        if c.loop_times:
            w["loop.in"], w["loop.step"] = mat(sd["loop.in"]), f32(sd["loop.step"])
        for i, l in enumerate(c.layers):
            p, x = f"l{i}.", f"l{i}.mix."
            w[p + "norm1"] = 1.0 + f32(sd[p + "norm1"])
            if l["type"] == "attention":
                w[x + "qkvg"] = mat(torch.cat([sd[x + "q"], sd[x + "k"], sd[x + "v"], sd[x + "g"]]))
                for k in ("q.norm", "k.norm", "r1", "r2"):
                    w[x + k] = f32(sd[x + k]).reshape(-1)
            elif l["type"] == "wkv":
                w[x + "mu"] = torch.stack([f32(sd[x + "mu." + s]) for s in "rkvgw"])
                for k in "rkvg":
                    w[x + k] = mat(sd[x + k])
                # w2 multiplies the fp32 tanh output: kept fp32 so that the fp32 product converts nothing per step
                w[x + "w1"], w[x + "w2"] = mat(sd[x + "w1"]), f32(sd[x + "w2"])
                for k in ("w0", "u", "norm"):
                    w[x + k] = f32(sd[x + k]).reshape(-1)
            else:
                w[x + "in"] = mat(torch.cat([sd[x + k] for k in ("q", "k", "v", "a1", "g1", "b")]))
                w[x + "conv"] = f32(torch.cat([sd[x + k + ".conv"] for k in "qkv"]))
                w[x + "a2"], w[x + "g2"] = mat(sd[x + "a2"]), mat(sd[x + "g2"])
                for k in ("A_log", "dt_bias", "norm"):
                    w[x + k] = f32(sd[x + k]).reshape(-1)
            w[x + "o"] = mat(sd[x + "o"])
            if l.get("mlp") is not None:
                w[p + "norm2"] = 1.0 + f32(sd[p + "norm2"])
                w[p + "mlp.up"], w[p + "mlp.down"] = mat(sd[p + "mlp.up"]), mat(sd[p + "mlp.down"])
                w[p + "mlp.act"] = f32(sd[p + "mlp.act"]).reshape(-1)
        self._alloc_state()
        return self

    load_hf_state = load_state

    def load_safetensors_dir(self, path: str):
        from safetensors.torch import load_file

        sd = {}
        for f in sorted(os.listdir(path)):
            if f.endswith(".safetensors"):
                sd.update(load_file(os.path.join(path, f)))
        return self.load_state(sd)

    def random_init(self, seed: int = 0):
        return self.load_state(random_state(self.cfg, seed))

    def num_params(self) -> int:
        return sum(t.numel() for t in self.w.values())

    # ------------------------------------------------------------------ recurrent state slots
    def _alloc_state(self):
        c = self.cfg
        self.pool.clear()
        self.state = {}
        for r in self.runs:
            l = c.layers[r[0]]
            m, tag = l["mixer"], f"l{r[0]}p{r[1]}."
            if l["type"] == "wkv":
                self.state[r] = dict(shift=self.pool.add(tag + "shift", (1, c.hidden_size)),
                                     S=self.pool.add(tag + "S", (m["heads"], m["dim"], m["dim"])))
            elif l["type"] == "channel_delta":
                C = 2 * m["kv_heads"] * m["dim"] + m["heads"] * m["vdim"]
                self.state[r] = dict(conv=self.pool.add(tag + "conv", (m["conv"] - 1, C)),
                                     S=self.pool.add(tag + "S", (m["heads"], m["dim"], m["vdim"])))

    def set_state_slots(self, n: int):
        """Engine hook: size the state pool for n live sequences (before any request is admitted)."""
        if n != self.pool.n_slots:
            self.pool = StatePool(n, self.device)
            if self.w:
                self._alloc_state()

    def release_request(self, sid: int):
        self.pool.release(sid)

    def prepare_batch(self, fb: ForwardBatch):
        """Engine hook: one (cu, slot, ctx, page table) row per sequence of the step - prompt portions first, then
        single decoded tokens - and fresh state for sequences that start at position 0."""
        P = len(fb.prefill_qlen)
        nd = fb.num_tokens - fb.num_prefill_tokens
        pctx = fb.prefill_ctx_host or []
        dctx = fb.decode_ctx_host or []
        sids = fb.seq_ids or []
        slots = [self.pool.slot(sid, pctx[i] == fb.prefill_qlen[i]) for i, sid in enumerate(sids[:P])]
        slots += [self.pool.slot(sid, dctx[j] == 1 if j < len(dctx) else False) for j, sid in enumerate(sids[P:])]
        cu = [0]
        for n in fb.prefill_qlen:
            cu.append(cu[-1] + n)
        cu += [cu[-1] + j + 1 for j in range(nd)]
        dev = self.device
        extra = dict(cu=torch.tensor(cu, dtype=torch.int32).to(dev, non_blocking=True),
                     slots=torch.tensor(slots, dtype=torch.int32).to(dev, non_blocking=True))
        parts_c = [t for t in (fb.prefill_ctx if P else None, fb.decode_ctx if nd else None) if t is not None]
        parts_b = [t for t in (fb.prefill_block_tables if P else None, fb.decode_block_tables if nd else None)
                   if t is not None]
        extra["ctx"] = parts_c[0] if len(parts_c) == 1 else torch.cat(parts_c)
        extra["bt"] = parts_b[0] if len(parts_b) == 1 else torch.cat(parts_b)
        fb.extra = extra

    def graph_static_inputs(self, bs: int) -> dict:
        """Static inputs of a captured decode graph of bs rows (the engine's ctx / page-table tensors complete them)."""
        return dict(cu=torch.arange(bs + 1, **self._i32), slots=torch.full((bs,), self.pool.pad_slot, **self._i32))

    def fill_graph_inputs(self, extra: dict, seq_ids, n: int):
        ids = torch.tensor([self.pool.slot(s, False) for s in seq_ids] +
                           [self.pool.pad_slot] * (extra["slots"].numel() - n), dtype=torch.int32)
        extra["slots"].copy_(ids, non_blocking=True)

    # ------------------------------------------------------------------ mixers
    def _attention(self, h, i, run, fb, kv, seq):
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        proj = ops.linear(h, w[x + "qkvg"])
        a, b, c = H * dk, H * dk + G * dk, H * dk + G * dk + G * dv
        kc, vc = kv.layer(self.kv_index[run])
        qn = ops.qknorm_kv_write(proj[:, :a], proj[:, a:b], proj[:, b:c], w[x + "q.norm"], w[x + "k.norm"], fb.slots,
                                 kc, vc, H, G, dk, dv, self.cfg.rms_eps)
        att = ops.window_attention(qn, kc, vc, seq["bt"], seq["cu"], seq["ctx"], H, G, dk, dv, float(m["scale"]),
                                   float(m.get("softcap") or 0.0), int((m.get("mask") or {}).get("size") or 0),
                                   w[x + "r1"], w[x + "r2"], gate=proj[:, c:])
        return ops.linear(att, w[x + "o"])

    def _wkv(self, h, i, run, seq):
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        H, d = m["heads"], m["dim"]
        st = self.state[run]
        T = h.shape[0]
        mixes = ops.token_shift_mix(h, w[x + "mu"], st["shift"].view(-1, h.shape[1]), seq["cu"], seq["slots"])
        ops.state_tail_write(h, st["shift"], seq["cu"], seq["slots"])
        rkv = torch.empty(3, T, H * d, dtype=self.dtype, device=h.device)
        for n, k in enumerate("rkv"):
            ops.linear(mixes[n], w[x + k], out=rkv[n])
        gate = ops.linear(mixes[3], w[x + "g"])
        lw = torch.tanh(ops.linear(mixes[4], w[x + "w1"], out_dtype=torch.float32))
        wpre = ops.linear(lw, w[x + "w2"], out_dtype=torch.float32)
        o = ops.wkv_scan(rkv[0], rkv[1], rkv[2], wpre, w[x + "w0"], w[x + "u"], st["S"], seq["cu"], seq["slots"])
        y = ops.head_norm_gate(o, gate, w[x + "norm"], "silu", self.cfg.rms_eps, self.dtype)
        return ops.linear(y, w[x + "o"])

    def _channel_delta(self, h, i, run, seq):
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        st = self.state[run]
        proj = ops.linear(h, w[x + "in"])
        C = 2 * G * dk + H * dv
        ra, rg = w[x + "a2"].shape[1], w[x + "g2"].shape[1]
        xc = proj[:, :C]
        y = ops.conv_silu(xc, w[x + "conv"], st["conv"], seq["cu"], seq["slots"])
        ops.state_tail_write(xc, st["conv"], seq["cu"], seq["slots"])
        a = ops.linear(proj[:, C:C + ra], w[x + "a2"], out_dtype=torch.float32)
        gate = ops.linear(proj[:, C + ra:C + ra + rg], w[x + "g2"])
        b = proj[:, C + ra + rg:].float()
        qn, kn, decay, beta = ops.delta_prep(y, a, b, w[x + "A_log"], w[x + "dt_bias"], H, G, dk)
        o = ops.delta_scan(qn, kn, y[:, 2 * G * dk:], decay, beta, st["S"], seq["cu"], seq["slots"], G)
        yy = ops.head_norm_gate(o, gate, w[x + "norm"], "sigmoid", self.cfg.rms_eps, self.dtype)
        return ops.linear(yy, w[x + "o"])

    # ------------------------------------------------------------------ forward
    def forward(self, fb: ForwardBatch, kv, decode_ws=None) -> torch.Tensor:
        """Returns fp32 logits [len(sample_rows), vocab]."""
        c, w, dt = self.cfg, self.w, self.dtype
        if fb.extra is None:  # direct forward without the engine hook
            self.prepare_batch(fb)
        seq = dict(fb.extra)
        if "ctx" not in seq:  # captured decode graph: one row per sequence, the engine's static ctx / page tables
            seq["ctx"], seq["bt"] = fb.decode_ctx, fb.decode_block_tables
        eps, mult = c.rms_eps, c.residual_mult
        x0 = ops.embed_scale_f32(fb.token_ids, w["embed"], c.embedding_scale)
        res, pend, x0c = x0, None, None
        if c.loop_times == 0 or c.loop_start > 0:
            res = x0.clone()
        for n, (i, t) in enumerate(self.runs):
            l = c.layers[i]
            p = f"l{i}."
            if c.loop_times and i == c.loop_start:
                xc = ops.add_rmsnorm_f32(res, pend, mult, None, eps, dt)
                pend = None
                if x0c is None:
                    x0c = x0.to(dt)
                res = ops.linear(torch.cat([xc, x0c], -1), w["loop.in"], out_dtype=torch.float32)
                res += w["loop.step"][t]
            h = ops.add_rmsnorm_f32(res, pend, mult, w[p + "norm1"], eps, dt)
            if l["type"] == "attention":
                pend = self._attention(h, i, (i, t), fb, kv, seq)
            elif l["type"] == "wkv":
                pend = self._wkv(h, i, (i, t), seq)
            else:
                pend = self._channel_delta(h, i, (i, t), seq)
            if l.get("mlp") is not None:
                h = ops.add_rmsnorm_f32(res, pend, mult, w[p + "norm2"], eps, dt)
                pend = ops.linear(ops.poly_norm(ops.linear(h, w[p + "mlp.up"]), w[p + "mlp.act"], eps),
                                  w[p + "mlp.down"])
            if self.capture_residuals is not None:
                if pend is not None:
                    ops.add_rmsnorm_f32(res, pend, mult)
                pend = None
                self.capture_residuals.append(res.clone())
        if fb.sample_rows is not None:
            res = res.index_select(0, fb.sample_rows)
            pend = pend.index_select(0, fb.sample_rows) if pend is not None else None
        xf = ops.add_rmsnorm_f32(res, pend, mult, w["final.norm"], eps, dt)
        return ops.linear(xf, w["head"], out_dtype=torch.float32)[:, : c.vocab_size]
