"""Ronavik: a hybrid decoder with post-norm gated residuals, whose layer list mixes two token mixers.

Architecture (every size and constant comes from ``config.json``; the layer list may hold the mixers in any order):
  * token embedding plus a learned absolute position vector (not scaled); the output head is the embedding table;
  * a layer is ``x += N1b(g1 * mixer(h))`` with ``h = N1(x)`` and ``g1 = sigmoid(W_rg1 h + b)``, then the same around
    the feed-forward (``N2``, ``N2b``, ``W_rg2``); all norms are plain-weight RMS norms; a layer may have no
    feed-forward;
  * mixer ``parallel``: two branches read the same ``h`` and their outputs add with fixed scales.
    ``left``: GQA without rotation and without softmax - q and k are RMS-normalised per head (one weight vector of the
    head size shared by the heads), the query at position p is multiplied by ``1 + coef ln(floor((p + 1) / every) + 1)``,
    a visible key weighs ``sigmoid(scale q.k + pb_h)``, causal. ``right``: a recurrent block ``W_o (S * gelu(W_y h))``
    with ``u = conv(W_x h)`` (short causal depthwise convolution), block-diagonal gates ``r, i = sigmoid(W u + b)``,
    ``a = exp(-8 r softplus(lam))`` and ``S <- a S + sqrt(1 - a^2) i u`` per channel;
  * mixer ``mamba2``: one input projection [z | x | B | C | dt]; x, B, C pass a short causal convolution + SiLU;
    ``dt = softplus(dt + dt_bias)``; per head ``S <- exp(-exp(A_log) dt) S + dt B x^T`` and ``y = S^T C + D x``;
    ``y * silu(z)`` is RMS-normalised in ``norm_groups`` parts, weighted, projected out;
  * feed-forward: mixture of experts with a sigmoid router; the chosen experts' scores (not renormalised) multiply
    each expert's INPUT; an expert is ``W_down relu(W_up .)^2``;
  * final RMS norm and the tied output head.

MI355X mapping: the residual stream, every norm statistic, attention scores and weights, positions, router scores,
decays, gates of the recurrences and the recurrent states are fp32; the projections run in the model dtype (bf16 on the
MFMA GEMMs with fp32 accumulation, or true fp32). The ``left`` branch keeps K / V in the engine's paged cache (one
cache layer per ``parallel`` layer, each with its own head geometry); the recurrent branches keep their fp32 states
(convolution tails, S vectors / matrices) in the engine's state slot pool. A step's rows - prompt portions and single
decoded tokens alike - go through the same HIP kernels, addressed by device-side (cu, slot, ctx) vectors, so
pure-decode steps replay a captured HIP graph. Per layer the projections that read the same input are one GEMM
(q | k | v | y | x | residual gate; in | residual gate), the two output projections of a
``parallel`` mixer are one GEMM over the concatenated branch outputs, and the closing norm of a sublayer is fused with
the residual add and the opening norm of the next sublayer.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from .. import ops
from ..engine.state_pool import StatePool
from ..parallel.dist import DistContext, get_context
from .common import ForwardBatch

MIXERS = ("parallel", "mamba2")
RGLRU_C = 8.0    # log a = -RGLRU_C * r * softplus(lam)


@dataclass
class RonavikConfig:
    vocab_size: int
    hidden_size: int
    layers: Tuple[dict, ...]                 # {"type", "mixer": {...}, "mlp": {"kind": "moe", ...} | None}
    max_position: int = 2048                 # rows of the learned position table
    rms_eps: float = 1e-6
    name: str = "ronavik"
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()

    def __post_init__(self):
        layers = []
        for i, l in enumerate(self.layers):
            if l["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
            m = dict(l["mixer"])
            if l["type"] == "parallel":
                a = dict(m["left"])
                a.setdefault("kv_heads", a["heads"])
                a.setdefault("vdim", a["dim"])
                a.setdefault("scale", a["dim"] ** -0.5)
                if a["heads"] % a["kv_heads"]:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                r = dict(m["right"])
                r.setdefault("blocks", 1)
                if r["width"] % r["blocks"]:
                    raise ValueError(f"layer {i}: the recurrent width must be a multiple of its blocks")
                m.update(left=a, right=r)
                m.setdefault("left_scale", 1.0)
                m.setdefault("right_scale", 1.0)
            else:
                m.setdefault("groups", 1)
                m.setdefault("norm_groups", 1)
                if m["heads"] % m["groups"] or (m["heads"] * m["vdim"]) % m["norm_groups"]:
                    raise ValueError(f"layer {i}: heads / groups / norm_groups do not divide")
            ml = l.get("mlp")
            if ml is not None:
                if ml.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {ml.get('kind')!r}")
                if not 1 <= ml["router"]["top"] <= min(8, ml["router"]["experts"]):
                    raise ValueError(f"layer {i}: 1 <= top <= min(8, experts)")
            layers.append(dict(l, mixer=m, mlp=ml))
        self.layers = tuple(layers)

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def head_dim(self) -> int:  # engine sizing hooks: the widest attention head
        return max([l["mixer"]["left"]["dim"] for l in self.layers if l["type"] == "parallel"] or [16])

    @staticmethod
    def from_json(path_or_dict) -> "RonavikConfig":
        if isinstance(path_or_dict, dict):
            c, name = path_or_dict, "ronavik"
        else:
            with open(os.path.join(path_or_dict, "config.json")) as f:
                c = json.load(f)
            name = os.path.basename(os.path.normpath(path_or_dict)) or "ronavik"
        eos = c.get("eos_token_id", ())
        return RonavikConfig(
            vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(c["layers"]),
            max_position=int(c.get("max_positions", 2048)), rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
            name=c.get("name", name), bos_token_id=c.get("bos_token_id"),
            eos_token_ids=tuple(eos) if isinstance(eos, (list, tuple)) else (eos,))

    @staticmethod
    def tiny(**kw) -> "RonavikConfig":
        par = dict(left=dict(dim=16, vdim=32, heads=4, kv_heads=2, scale=0.3, q_temp=dict(coef=0.4, every=8)),
                   right=dict(width=48, blocks=3, conv=3), left_scale=0.8, right_scale=1.3)
        ssm = dict(heads=4, vdim=16, state=16, groups=2, norm_groups=2, conv=4)
        mlp = dict(kind="moe", expert=dict(ff=64), router=dict(experts=4, top=2))
        base = dict(vocab_size=512, hidden_size=64, name="tiny-ronavik", rms_eps=1e-5, max_position=512,
                    layers=(dict(type="mamba2", mixer=ssm, mlp=mlp), dict(type="parallel", mixer=par, mlp=mlp),
                            dict(type="parallel", mixer=par, mlp=None), dict(type="mamba2", mixer=ssm, mlp=mlp)))
        base.update(kw)
        return RonavikConfig(**base)

    @staticmethod
    def sized(width: int, n_layers: int, ff: int, heads: int, head_dim: int, experts: int = 8, top: int = 2,
              vocab: int = 32768, max_position: int = 8192, pattern: Tuple[str, ...] = MIXERS, **kw) -> "RonavikConfig":
        """A regular stack for benchmarks: `pattern` repeated over n_layers, equal head geometry in every mixer."""
        mix = dict(parallel=dict(left=dict(dim=head_dim, vdim=head_dim, heads=heads, kv_heads=max(1, heads // 4),
                                           scale=head_dim ** -0.5, q_temp=dict(coef=0.1, every=1024)),
                                 right=dict(width=width, blocks=max(1, width // 256), conv=4),
                                 left_scale=1.0, right_scale=1.0),
                   mamba2=dict(heads=2 * width // head_dim if head_dim <= 64 else 2 * width // 64, vdim=min(head_dim, 64),
                               state=128, groups=max(1, heads // 8), norm_groups=max(1, heads // 8), conv=4))
        mix["mamba2"]["heads"] -= mix["mamba2"]["heads"] % mix["mamba2"]["groups"]
        layers = tuple(dict(type=pattern[i % len(pattern)], mixer=mix[pattern[i % len(pattern)]],
                            mlp=dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top)))
                       for i in range(n_layers))
        base = dict(vocab_size=vocab, hidden_size=width, layers=layers, max_position=max_position,
                    name=f"ronavik-{width}x{n_layers}")
        base.update(kw)
        return RonavikConfig(**base)


def random_state(cfg: RonavikConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """A random checkpoint (tensor names and shapes of the safetensors layout, fp32 values) with magnitudes that keep
    activations, decays and states in a trained model's range."""
    g = torch.Generator().manual_seed(seed)
    D = cfg.hidden_size
    rn = lambda *s, std=1.0: torch.randn(*s, generator=g) * std  # noqa: E731
    un = lambda *s, lo=0.0, hi=1.0: torch.rand(*s, generator=g) * (hi - lo) + lo  # noqa: E731
    lin = lambda o, i: rn(o, i, std=i ** -0.5)  # noqa: E731
    sd: Dict[str, torch.Tensor] = {"embed": rn(cfg.vocab_size, D), "pos": rn(cfg.max_position, D, std=0.3),
                                   "final.norm": 1 + rn(D, std=0.1)}
    for i, l in enumerate(cfg.layers):
        p, m, x = f"l{i}.", l["mixer"], f"l{i}.mix."
        for k in ("norm1", "norm1b"):
            sd[p + k] = 1 + rn(D, std=0.1)
        sd[p + "rg1"], sd[p + "rg1.b"] = lin(D, D), rn(D, std=0.5)
        if l["type"] == "parallel":
            a, r = m["left"], m["right"]
            H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            xl, xr = x + "left.", x + "right."
            sd[xl + "q"], sd[xl + "k"], sd[xl + "v"] = lin(H * dk, D), lin(G * dk, D), lin(G * dv, D)
            sd[xl + "q.norm"], sd[xl + "k.norm"] = 1 + rn(dk, std=0.1), 1 + rn(dk, std=0.1)
            sd[xl + "pb"] = un(H, lo=-4.0, hi=-1.0)
            sd[xl + "o"] = lin(D, H * dv)
            W, nb, K = r["width"], r["blocks"], r["conv"]
            bs = W // nb
            sd[xr + "y"], sd[xr + "y.b"] = lin(W, D), rn(W, std=0.2)
            sd[xr + "x"], sd[xr + "x.b"] = lin(W, D), rn(W, std=0.2)
            sd[xr + "conv"], sd[xr + "conv.b"] = rn(W, K, std=K ** -0.5), rn(W, std=0.1)
            sd[xr + "ra"], sd[xr + "ra.b"] = rn(nb, bs, bs, std=bs ** -0.5), rn(nb, bs, std=0.5)
            sd[xr + "ri"], sd[xr + "ri.b"] = rn(nb, bs, bs, std=bs ** -0.5), rn(nb, bs, std=0.5)
            sd[xr + "lam"] = un(W, lo=-4.0, hi=0.0)
            sd[xr + "o"] = lin(D, W)
        else:
            H, dv, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            inner, C = H * dv, H * dv + 2 * G * N
            sd[x + "in"] = lin(2 * inner + 2 * G * N + H, D)
            sd[x + "conv"], sd[x + "conv.b"] = rn(C, K, std=K ** -0.5), rn(C, std=0.1)
            sd[x + "dt_bias"] = un(H, lo=-3.0, hi=0.5)
            sd[x + "A_log"] = torch.log(un(H, lo=0.5, hi=4.0))
            sd[x + "D"] = 1 + rn(H, std=0.2)
            sd[x + "norm"] = 1 + rn(inner, std=0.1)
            sd[x + "o"] = lin(D, inner)
        ml = l.get("mlp")
        if ml is not None:
            F_, E = ml["expert"]["ff"], ml["router"]["experts"]
            for k in ("norm2", "norm2b"):
                sd[p + k] = 1 + rn(D, std=0.1)
            sd[p + "rg2"], sd[p + "rg2.b"] = lin(D, D), rn(D, std=0.5)
            sd[p + "mlp.router"] = lin(E, D) * 2.0
            for e in range(E):
                sd[p + f"mlp.e{e}.up"], sd[p + f"mlp.e{e}.down"] = lin(F_, D) * 1.5, lin(D, F_)
    return sd


class RonavikModel:
    """Weights (plain tensors) + forward for the serving engine (the hooks of LlamaModel / PinavikModel)."""

    has_recurrent_state = True       # no prefix-cache reuse: a cached prefix has no recurrent state to resume from
    attention_backend = "window"     # the paged window / sigmoid attention kernels: no flash-attention tile lists

    def __init__(self, cfg: RonavikConfig, device=None, dtype=torch.bfloat16, dist_ctx: DistContext | None = None,
                 state_slots: Optional[int] = None):
        self.cfg = cfg
        self.ctx = dist_ctx or get_context()
        assert self.ctx.tp_size == 1, "Ronavik runs TP=1"
        self.device = torch.device(device) if device is not None else self.ctx.device
        self.dtype = dtype
        att = [i for i, l in enumerate(cfg.layers) if l["type"] == "parallel"]
        self.kv_index = {i: j for j, i in enumerate(att)}
        self.num_kv_layers = len(att)
        heads = [cfg.layers[i]["mixer"]["left"] for i in att]
        self.hq = max([m["heads"] for m in heads] or [1])
        self.hkv = max([m["kv_heads"] for m in heads] or [1])
        self.vocab_local, self.vstart = cfg.vocab_size, 0
        self.lora_names: list = []
        self.w: Dict[str, torch.Tensor] = {}
        self.pool = StatePool(state_slots or int(os.environ.get("GAI_LINEAR_STATE_SLOTS", "64")), self.device)
        self.state: Dict[int, Dict[str, torch.Tensor]] = {}
        self.capture_residuals: Optional[list] = None  # numerics debugging: the residual stream after every layer
        self._i32 = dict(dtype=torch.int32, device=self.device)

    # ------------------------------------------------------------------ engine sizing hooks
    def kv_layout(self) -> List[Tuple[int, int, int]]:
        """(kv heads, key size, value size) of every paged cache layer: one per `parallel` layer."""
        out = []
        for i in sorted(self.kv_index, key=self.kv_index.get):
            m = self.cfg.layers[i]["mixer"]["left"]
            out.append((m["kv_heads"], m["dim"], m["vdim"]))
        return out

    # ------------------------------------------------------------------ weights
    def load_state(self, sd: Dict[str, torch.Tensor]):
        """Checkpoint tensors (the safetensors names) -> device weights: projections in the model dtype, per-channel
        tables and the block-diagonal gate matrices fp32, same-input projections fused."""
        c, dev, dt = self.cfg, self.device, self.dtype
        f32 = lambda t: t.to(torch.float32).to(dev).contiguous()  # noqa: E731
        mat = lambda t: t.to(torch.float32).to(dev, dt).contiguous()  # noqa: E731
        D = c.hidden_size
        w = self.w = {}
        w["embed"], w["pos"] = mat(sd["embed"]), mat(sd["pos"])
        w["final.norm"] = f32(sd["final.norm"])
        for i, l in enumerate(c.layers):
            p, x, m = f"l{i}.", f"l{i}.mix.", l["mixer"]
            for k in ("norm1", "norm1b"):
                w[p + k] = f32(sd[p + k])
            if l["type"] == "parallel":
                xl, xr = x + "left.", x + "right."
                a, r = m["left"], m["right"]
                nqkv = (a["heads"] + a["kv_heads"]) * a["dim"] + a["kv_heads"] * a["vdim"]
                w[x + "in"] = mat(torch.cat([sd[xl + "q"], sd[xl + "k"], sd[xl + "v"], sd[xr + "y"], sd[xr + "x"],
                                             sd[p + "rg1"]]))
                w[x + "in.b"] = mat(torch.cat([torch.zeros(nqkv), sd[xr + "y.b"].float(), sd[xr + "x.b"].float(),
                                               sd[p + "rg1.b"].float()]))
                for k in ("q.norm", "k.norm", "pb"):
                    w[xl + k] = f32(sd[xl + k]).reshape(-1)
                w[xr + "conv"], w[xr + "conv.b"] = f32(sd[xr + "conv"]), f32(sd[xr + "conv.b"])
                # gate matrices [blocks, out, in] -> [blocks, in, out]: the kernel's threads own output channels
                w[xr + "ra"], w[xr + "ri"] = f32(sd[xr + "ra"].transpose(1, 2)), f32(sd[xr + "ri"].transpose(1, 2))
                w[xr + "ra.b"], w[xr + "ri.b"] = f32(sd[xr + "ra.b"]).reshape(-1), f32(sd[xr + "ri.b"]).reshape(-1)
                w[xr + "lam"] = f32(sd[xr + "lam"])
                w[x + "o"] = mat(torch.cat([sd[xl + "o"], sd[xr + "o"]], 1))
            else:
                w[x + "in"] = mat(torch.cat([sd[x + "in"], sd[p + "rg1"]]))
                w[x + "in.b"] = mat(torch.cat([torch.zeros(sd[x + "in"].shape[0]), sd[p + "rg1.b"].float()]))
                w[x + "conv"], w[x + "conv.b"] = f32(sd[x + "conv"]), f32(sd[x + "conv.b"])
                for k in ("dt_bias", "A_log", "D", "norm"):
                    w[x + k] = f32(sd[x + k]).reshape(-1)
                w[x + "o"] = mat(sd[x + "o"])
            ml = l.get("mlp")
            if ml is not None:
                E = ml["router"]["experts"]
                for k in ("norm2", "norm2b"):
                    w[p + k] = f32(sd[p + k])
                w[p + "rg2"], w[p + "rg2.b"] = mat(sd[p + "rg2"]), mat(sd[p + "rg2.b"])
                # router rows padded to the GEMM's 16-column grid: the logits come out of the MFMA kernel in fp32
                pad = (-E) % 16
                w[p + "mlp.router"] = mat(torch.cat([sd[p + "mlp.router"].float(), torch.zeros(pad, D)]))
                w[p + "mlp.up"] = mat(torch.stack([sd[p + f"mlp.e{e}.up"] for e in range(E)]))
                w[p + "mlp.down"] = mat(torch.stack([sd[p + f"mlp.e{e}.down"] for e in range(E)]))
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
        self.pool.clear()
        self.state = {}
        for i, l in enumerate(self.cfg.layers):
            m, tag = l["mixer"], f"l{i}."
            if l["type"] == "parallel":
                r = m["right"]
                self.state[i] = dict(conv=self.pool.add(tag + "conv", (r["conv"] - 1, r["width"])),
                                     S=self.pool.add(tag + "S", (r["width"],)))
            else:
                C = m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"]
                self.state[i] = dict(conv=self.pool.add(tag + "conv", (m["conv"] - 1, C)),
                                     S=self.pool.add(tag + "S", (m["heads"], m["state"], m["vdim"])))

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
    def _parallel(self, h, i, fb, kv, seq):
        """-> (mixer output, residual-gate logits)."""
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        a, r = m["left"], m["right"]
        H, G, dk, dv, W = a["heads"], a["kv_heads"], a["dim"], a["vdim"], r["width"]
        xl, xr = x + "left.", x + "right."
        proj = ops.linear(h, w[x + "in"], w[x + "in.b"])
        c0 = H * dk
        c1 = c0 + G * dk
        c2 = c1 + G * dv
        c3, c4 = c2 + W, c2 + 2 * W
        T = h.shape[0]
        both = torch.empty(T, H * dv + W, dtype=self.dtype, device=h.device)
        # left: sigmoid attention over the paged cache
        kc, vc = kv.layer(self.kv_index[i])
        qt = a.get("q_temp") or {}
        qn = ops.headnorm_kv_write(proj[:, :c0], proj[:, c0:c1], proj[:, c1:c2], w[xl + "q.norm"], w[xl + "k.norm"],
                                   fb.slots, kc, vc, H, G, dk, dv, self.cfg.rms_eps, fb.positions,
                                   float(qt.get("coef") or 0.0), int(qt.get("every") or 1))
        ops.sigmoid_attention(qn, kc, vc, seq["bt"], seq["cu"], seq["ctx"], H, G, dk, dv, float(a["scale"]),
                              w[xl + "pb"], out=both[:, : H * dv], out_scale=float(m["left_scale"]))
        # right: gated linear recurrence over the convolved x branch
        st = self.state[i]
        xb = proj[:, c3:c4]
        u = ops.conv_silu(xb, w[xr + "conv"], st["conv"], seq["cu"], seq["slots"], bias=w[xr + "conv.b"], act=False)
        ops.state_tail_write(xb, st["conv"], seq["cu"], seq["slots"])
        ga, gb = ops.rglru_gates(u, w[xr + "ra"], w[xr + "ra.b"], w[xr + "ri"], w[xr + "ri.b"], w[xr + "lam"], RGLRU_C)
        ops.rglru_scan(ga, gb, proj[:, c2:c3], st["S"], seq["cu"], seq["slots"], self.dtype, act="gelu_tanh",
                       out=both[:, H * dv:], out_scale=float(m["right_scale"]))
        return ops.linear(both, w[x + "o"]), proj[:, c4:]

    def _mamba2(self, h, i, seq):
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        H, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
        inner, gn = H * dv, G * N
        st = self.state[i]
        proj = ops.linear(h, w[x + "in"], w[x + "in.b"])
        c1 = 2 * inner + 2 * gn
        xbc = proj[:, inner:c1]
        cv = ops.conv_silu(xbc, w[x + "conv"], st["conv"], seq["cu"], seq["slots"], bias=w[x + "conv.b"], act=True)
        ops.state_tail_write(xbc, st["conv"], seq["cu"], seq["slots"])
        y = ops.ssd_scan(cv[:, :inner], cv[:, inner:inner + gn], cv[:, inner + gn:], proj[:, c1:c1 + H], w[x + "dt_bias"],
                         w[x + "A_log"], w[x + "D"], st["S"], seq["cu"], seq["slots"], G)
        yn = ops.gate_group_norm(y.view(-1, inner), proj[:, :inner], w[x + "norm"], m["norm_groups"], self.cfg.rms_eps,
                                 self.dtype)
        return ops.linear(yn, w[x + "o"]), proj[:, c1 + H:]

    def _moe(self, h, i):
        """-> (feed-forward output, residual-gate logits)."""
        ml, w, p = self.cfg.layers[i]["mlp"], self.w, f"l{i}."
        D, E, top = self.cfg.hidden_size, ml["router"]["experts"], ml["router"]["top"]
        gate = ops.linear(h, w[p + "rg2"], w[p + "rg2.b"])
        logits = ops.linear(h, w[p + "mlp.router"], out_dtype=torch.float32)[:, :E]
        ids, wts = ops.moe_route(logits, top, renorm=False, score="sigmoid")
        _rows, offs, pos = ops.moe_dispatch(ids, E)
        xs = ops.moe_scale_rows(h, pos, wts)
        n = h.shape[0] * top
        up = ops.moe_gemm(xs, None, w[p + "mlp.up"], offs, n, act="relu2")
        dn = ops.moe_gemm(up, None, w[p + "mlp.down"], offs, n)
        return ops.moe_combine(dn, pos, None), gate

    # ------------------------------------------------------------------ forward
    def forward(self, fb: ForwardBatch, kv, decode_ws=None) -> torch.Tensor:
        """Returns fp32 logits [len(sample_rows), vocab]."""
        c, w, dt = self.cfg, self.w, self.dtype
        if fb.extra is None:  # direct forward without the engine hook
            self.prepare_batch(fb)
        seq = dict(fb.extra)
        if "ctx" not in seq:  # captured decode graph: one row per sequence, the engine's static ctx / page tables
            seq["ctx"], seq["bt"] = fb.decode_ctx, fb.decode_block_tables
        eps, L = c.rms_eps, len(c.layers)
        res = ops.embed_scale_f32(fb.token_ids, w["embed"], 1.0, fb.positions, w["pos"])
        h = ops.add_rmsnorm_f32(res, None, 1.0, w["l0.norm1"], eps, dt) if L else None
        for i, l in enumerate(c.layers):
            p = f"l{i}."
            y, gate = self._parallel(h, i, fb, kv, seq) if l["type"] == "parallel" else self._mamba2(h, i, seq)
            last = i + 1 == L
            nxt = None if last else w[f"l{i + 1}.norm1"]
            if l.get("mlp") is not None:
                h = ops.gated_norm_add_f32(res, y, gate, w[p + "norm1b"], eps, w[p + "norm2"], dt)
                y, gate = self._moe(h, i)
                h = ops.gated_norm_add_f32(res, y, gate, w[p + "norm2b"], eps, nxt, None if last else dt)
            else:
                h = ops.gated_norm_add_f32(res, y, gate, w[p + "norm1b"], eps, nxt, None if last else dt)
            if self.capture_residuals is not None:
                self.capture_residuals.append(res.clone())
        if fb.sample_rows is not None:
            res = res.index_select(0, fb.sample_rows)
        xf = ops.add_rmsnorm_f32(res, None, 1.0, w["final.norm"], eps, dt)
        return ops.linear(xf, w["embed"], out_dtype=torch.float32)[:, : c.vocab_size]
