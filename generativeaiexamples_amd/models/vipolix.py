"""Vipolix: a hybrid decoder whose layer list mixes gated linear attention with a layer that runs chunk-local attention
and a generalised delta rule side by side, with token shift in front of every mixer, mixture-of-experts feed-forwards
and a per-layer token input.

Architecture (every size and constant comes from ``config.json``; the layer list may hold the mixers in any order):
  * token embedding; the output head is its own matrix;
  * a layer is pre-norm: ``x += mixer(shift(N1(x)))`` then ``x += ff(N2(x))``; the norm is an RMS norm with a
    zero-centred weight (``* (1 + w)``); a layer may have no feed-forward;
  * token shift: the mixer reads ``h_t + (h_(t-1) - h_t) * mu`` (zeros before the first token);
  * per-layer token input, after the feed-forward: the layer's slice e of a second embedding of the token,
    ``y = W_proj (gelu_tanh(W_gate x) * e)``, ``x += rmsnorm(y) * w``;
  * mixer ``gla``: gated linear attention ``S <- diag(alpha) S + k v^T, o = S^T q`` with a decay per key channel
    ``alpha = sigmoid(z)^(1 / tau)`` from a low-rank projection; per-head RMS norm (one weight vector shared by the
    heads), a SiLU gate;
  * mixer ``parallel``: two branches on the same input, added with fixed scales. Left: GQA with biases and a short
    causal convolution on q, k and v, a rotation of the first ``rot.dims`` channels of each head in interleaved pairs,
    a temperature per head, keys visible only inside the query's own chunk of ``mask.size`` positions, and a softmax
    whose denominator carries an extra 1 (a value-less sink of score 0). Right: the generalised delta rule ``S <- diag(w) S - (a * u)(u^T S) + k v^T``
    with the unit key u, decay ``w = exp(-e^(-1/2) sigmoid(.))`` and removal rate ``a = sigmoid(.)`` per key channel;
    per-head unit RMS, a weight over all heads, a sigmoid gate;
  * feed-forward: a mixture of experts with a sigmoid router - the choice made on ``score + correction`` among the
    experts of the best groups, the weights the plain scores renormalised and scaled - over experts
    ``W_down (g sigmoid(1.702 g) (u + 1))`` with ``g = min(W_gate h, limit)``, ``u = clamp(W_up h, +-limit)``, plus a
    shared expert of the same form times ``sigmoid(w_sg . h)``.

MI355X mapping. The residual stream, norms, positions and angles, attention scores and weights, router, decays, removal
rates, unit keys and recurrent states are fp32; projections run in the model dtype (bf16 MFMA GEMMs with fp32
accumulation, or true fp32). K / V pages come from the engine's paged cache (one layer per ``parallel`` layer, with
that layer's kv heads and head sizes); recurrent states, convolution tails and the token-shift rows live in the engine's
state slot pool. A step's rows - prompt portions and single decoded tokens alike - go through the same HIP kernels,
addressed by device-side (cu, slot, ctx) vectors, so pure-decode steps replay a captured HIP graph. Both recurrences run
on one scan kernel (diagonal decay plus an optional rank-one removal); the chunk mask, the sink and the per-head
temperature are modes of the paged window-attention kernels.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from .. import ops
from ..engine.state_pool import StatePool
from ..parallel.dist import DistContext, get_context
from .common import ForwardBatch

MIXERS = ("gla", "parallel")
ROUTE_EPS = 1e-20               # added to the sum of the chosen router scores
UNIT_EPS = 1e-6                 # inside the root of the delta rule's unit key
DECAY_RATE = math.exp(-0.5)     # w = exp(-DECAY_RATE * sigmoid(.))
SINK_SCORE = 0.0                # the softmax denominator gains exp(0) = 1


@dataclass
class VipolixConfig:
    vocab_size: int
    hidden_size: int
    layers: Tuple[dict, ...]                 # {"type", "mixer": {...}, "mlp": {"kind": "moe", ...} | None}
    rms_eps: float = 1e-6
    side_dim: int = 0                        # 0: no per-layer token input
    name: str = "vipolix"
    max_position: int = 1 << 20              # angles are computed from the position: no table to outgrow
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()

    def __post_init__(self):
        layers = []
        for i, l in enumerate(self.layers):
            if l["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
            m = dict(l["mixer"])
            if l["type"] == "gla":
                m.setdefault("vdim", m["dim"])
                m.setdefault("tau", 1.0)
            else:
                a, r = dict(m["left"]), dict(m["right"])
                a.setdefault("kv_heads", a["heads"])
                a.setdefault("vdim", a["dim"])
                a.setdefault("scale", a["dim"] ** -0.5)
                a["conv"] = int(a.get("conv") or 0)
                rot = dict(a.get("rot") or {})
                dims = int(rot.setdefault("dims", 0) or 0)
                rot.setdefault("base", 10000.0)
                if dims % 2 or not 0 <= dims <= a["dim"]:
                    raise ValueError(f"layer {i}: the rotation covers an even number of a head's channels")
                if a["heads"] % a["kv_heads"]:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                a["rot"] = rot
                m.update(left=a, right=r)
                m.setdefault("left_scale", 1.0)
                m.setdefault("right_scale", 1.0)
            ml = l.get("mlp")
            if ml is not None:
                ml = dict(ml)
                if ml.setdefault("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {ml['kind']!r}")
                r = dict(ml["router"])
                g = dict(r.get("groups") or {})
                g.setdefault("count", 1)
                g.setdefault("keep", g["count"])
                r["groups"] = g
                r.setdefault("scale", 1.0)
                if r["experts"] % g["count"] or not 1 <= g["keep"] <= g["count"]:
                    raise ValueError(f"layer {i}: experts form groups.count equal groups, 1 <= keep <= count")
                if not 1 <= r["top"] <= min(16, r["experts"] // g["count"] * g["keep"]):
                    raise ValueError(f"layer {i}: 1 <= top <= min(16, experts of the kept groups)")
                ml["router"] = r
            layers.append(dict(l, mixer=m, mlp=ml))
        self.layers = tuple(layers)

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def head_dim(self) -> int:  # engine sizing hooks: the widest cached key row
        return max([l["mixer"]["left"]["dim"] for l in self.layers if l["type"] == "parallel"] or [16])

    @staticmethod
    def from_json(path_or_dict) -> "VipolixConfig":
        if isinstance(path_or_dict, dict):
            c, name = path_or_dict, "vipolix"
        else:
            with open(os.path.join(path_or_dict, "config.json")) as f:
                c = json.load(f)
            name = os.path.basename(os.path.normpath(path_or_dict)) or "vipolix"
        eos = c.get("eos_token_id", ())
        return VipolixConfig(
            vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(c["layers"]),
            rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)), side_dim=int((c.get("token_side") or {}).get("dim") or 0),
            name=c.get("name", name), max_position=int(c.get("max_position", 1 << 20)),
            bos_token_id=c.get("bos_token_id"), eos_token_ids=tuple(eos) if isinstance(eos, (list, tuple)) else (eos,))

    @staticmethod
    def tiny(**kw) -> "VipolixConfig":
        gla = dict(heads=2, dim=16, vdim=24, tau=8.0)
        par = dict(left=dict(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, scale=0.3, mask=dict(size=20),
                             rot=dict(base=10000.0, dims=8)),
                   right=dict(heads=2, dim=16), left_scale=0.7, right_scale=1.2)
        moe = dict(kind="moe", expert=dict(ff=32, limit=2.0), shared=dict(ff=48, limit=3.0),
                   router=dict(experts=6, top=2, scale=1.3, groups=dict(count=3, keep=2)))
        base = dict(vocab_size=512, hidden_size=64, name="tiny-vipolix", rms_eps=1e-5, side_dim=8,
                    layers=(dict(type="gla", mixer=gla, mlp=moe), dict(type="parallel", mixer=par, mlp=moe),
                            dict(type="parallel", mixer=par, mlp=None), dict(type="gla", mixer=gla, mlp=moe)))
        base.update(kw)
        return VipolixConfig(**base)

    @staticmethod
    def sized(width: int, n_layers: int, ff: int, heads: int, head_dim: int, chunk: int = 1024, vocab: int = 32768,
              experts: int = 8, top: int = 2, pattern: Tuple[str, ...] = MIXERS, **kw) -> "VipolixConfig":
        """A regular stack for benchmarks: `pattern` repeated over n_layers; every layer carries `experts` experts of
        ff / top (the active routed feed-forward equals a dense ff) plus a shared expert of ff / 4."""
        mix = dict(gla=dict(heads=heads, dim=head_dim, vdim=head_dim, tau=8.0),
                   parallel=dict(left=dict(heads=heads, kv_heads=max(1, heads // 4), dim=head_dim, vdim=head_dim, conv=4,
                                           scale=head_dim ** -0.5, mask=dict(size=chunk),
                                           rot=dict(base=10000.0, dims=head_dim // 2)),
                                 right=dict(heads=max(1, heads // 2), dim=head_dim), left_scale=1.0, right_scale=1.0))
        moe = dict(kind="moe", expert=dict(ff=ff // top, limit=7.0), shared=dict(ff=ff // 4, limit=7.0),
                   router=dict(experts=experts, top=top, scale=1.0, groups=dict(count=min(4, experts), keep=min(2, experts))))
        layers = tuple(dict(type=pattern[i % len(pattern)], mixer=mix[pattern[i % len(pattern)]], mlp=moe)
                       for i in range(n_layers))
        base = dict(vocab_size=vocab, hidden_size=width, layers=layers, side_dim=64, name=f"vipolix-{width}x{n_layers}")
        base.update(kw)
        return VipolixConfig(**base)


def random_state(cfg: VipolixConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """A random checkpoint (tensor names and shapes of the safetensors layout, fp32 values) with magnitudes that keep
    activations, decays and states in a trained model's range."""
    g = torch.Generator().manual_seed(seed)
    D = cfg.hidden_size
    rn = lambda *s, std=1.0: torch.randn(*s, generator=g) * std  # noqa: E731
    un = lambda *s, lo=0.0, hi=1.0: torch.rand(*s, generator=g) * (hi - lo) + lo  # noqa: E731
    lin = lambda o, i: rn(o, i, std=i ** -0.5)  # noqa: E731
    sd: Dict[str, torch.Tensor] = {"embed": rn(cfg.vocab_size, D), "head": lin(cfg.vocab_size, D) * 2.0,
                                   "final.norm": rn(D, std=0.1)}
    if cfg.side_dim:
        sd["side.embed"] = rn(cfg.vocab_size, cfg.num_layers * cfg.side_dim)

    def gated(p, F_):
        sd[p + "gate"], sd[p + "up"], sd[p + "down"] = lin(F_, D) * 1.5, lin(F_, D) * 1.5, lin(D, F_)

    for i, l in enumerate(cfg.layers):
        p, m, x = f"l{i}.", l["mixer"], f"l{i}.mix."
        sd[p + "norm1"], sd[p + "shift"] = rn(D, std=0.1), un(D, lo=0.0, hi=0.8)
        if l["type"] == "gla":
            H, dk, dv, lr = m["heads"], m["dim"], m["vdim"], max(4, D // 16)
            sd[x + "q"], sd[x + "k"], sd[x + "v"] = lin(H * dk, D) * 2.0, lin(H * dk, D), lin(H * dv, D)
            sd[x + "g"], sd[x + "o"] = lin(H * dv, D), lin(D, H * dv)
            sd[x + "norm"] = 1 + rn(dv, std=0.1)
            sd[x + "a1"], sd[x + "a2"], sd[x + "a2.b"] = lin(lr, D), lin(H * dk, lr) * 2.0, un(H * dk, lo=0.0, hi=4.0)
        else:
            a, r = m["left"], m["right"]
            H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            xl, xr = x + "left.", x + "right."
            for n, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
                sd[xl + n], sd[xl + n + ".b"] = lin(rows, D) * (2.0 if n != "v" else 1.0), rn(rows, std=0.1)
                if a["conv"]:
                    sd[xl + n + ".conv"] = rn(rows, a["conv"], std=0.3) + torch.eye(a["conv"])[-1]
            sd[xl + "temp"], sd[xl + "o"] = un(H, lo=0.6, hi=1.5), lin(D, H * dv)
            Hr, d, lr = r["heads"], r["dim"], max(4, D // 16)
            for n in ("r", "k", "v", "g", "a"):
                sd[xr + n] = lin(Hr * d, D)
            sd[xr + "a.b"] = rn(Hr * d, std=0.5)
            sd[xr + "w1"], sd[xr + "w2"], sd[xr + "w0"] = lin(lr, D), lin(Hr * d, lr) * 2.0, un(Hr * d, lo=-4.0, hi=0.0)
            sd[xr + "norm"], sd[xr + "o"] = 1 + rn(Hr * d, std=0.1), lin(D, Hr * d)
        ml = l.get("mlp")
        if ml is not None:
            sd[p + "norm2"] = rn(D, std=0.1)
            r = ml["router"]
            for e in range(r["experts"]):
                gated(p + f"mlp.e{e}.", ml["expert"]["ff"])
            sd[p + "mlp.router"] = lin(r["experts"], D) * 2.0
            sd[p + "mlp.correction"] = rn(r["experts"], std=0.1)
            if ml.get("shared"):
                gated(p + "mlp.shared.", ml["shared"]["ff"])
                sd[p + "mlp.shared.sg"] = lin(1, D)
        if cfg.side_dim:
            sd[p + "side.gate"], sd[p + "side.proj"] = lin(cfg.side_dim, D), lin(D, cfg.side_dim)
            sd[p + "side.norm"] = rn(D, std=0.3)
    return sd


class VipolixModel:
    """Weights (plain tensors) + forward for the serving engine (the hooks of LlamaModel / PinavikModel)."""

    has_recurrent_state = True       # no prefix-cache reuse: a cached prefix has no recurrent state to resume from
    attention_backend = "window"     # the paged window attention kernels: no flash-attention tile lists

    def __init__(self, cfg: VipolixConfig, device=None, dtype=torch.bfloat16, dist_ctx: DistContext | None = None,
                 state_slots: Optional[int] = None):
        self.cfg = cfg
        self.ctx = dist_ctx or get_context()
        assert self.ctx.tp_size == 1, "Vipolix runs TP=1"
        self.device = torch.device(device) if device is not None else self.ctx.device
        self.dtype = dtype
        att = [i for i, l in enumerate(cfg.layers) if l["type"] == "parallel"]
        self.kv_index = {i: j for j, i in enumerate(att)}
        self.num_kv_layers = len(att)
        self.hq = max([cfg.layers[i]["mixer"]["left"]["heads"] for i in att] or [1])
        self.hkv = max([cfg.layers[i]["mixer"]["left"]["kv_heads"] for i in att] or [1])
        self.vocab_local, self.vstart = cfg.vocab_size, 0
        self.lora_names: list = []
        self.w: Dict[str, torch.Tensor] = {}
        self.shared_gated: set = set()   # layers whose shared expert has a per-token sigmoid gate
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
        tables fp32, same-input projections fused, norm weights stored as 1 + w, expert matrices stacked with gate /
        up rows interleaved per 16 (rows padded with zeros to the grouped GEMM's grid: a zero gate / up row contributes
        nothing)."""
        c, dev, dt = self.cfg, self.device, self.dtype
        f32 = lambda t: t.to(torch.float32).to(dev).contiguous()  # noqa: E731
        mat = lambda t: t.to(torch.float32).to(dev, dt).contiguous()  # noqa: E731
        D = c.hidden_size
        pad16 = lambda t: torch.cat([t.float(), torch.zeros((-t.shape[0]) % 16, t.shape[1])])  # noqa: E731
        w = self.w = {}
        w["embed"], w["head"] = mat(sd["embed"]), mat(sd["head"])
        w["final.norm"] = f32(1 + sd["final.norm"].float())
        if c.side_dim:
            w["side.embed"] = mat(sd["side.embed"])
        for i, l in enumerate(c.layers):
            p, x, m = f"l{i}.", f"l{i}.mix.", l["mixer"]
            w[p + "norm1"] = f32(1 + sd[p + "norm1"].float())
            if p + "shift" in sd:
                w[p + "shift"] = f32(sd[p + "shift"]).reshape(1, D)
            if l["type"] == "gla":
                w[x + "in"] = mat(pad16(torch.cat([sd[x + k].float() for k in ("q", "k", "v", "g", "a1")])))
                w[x + "a2"], w[x + "a2.b"] = mat(sd[x + "a2"]), f32(sd[x + "a2.b"])
                w[x + "norm"] = f32(sd[x + "norm"])
                w[x + "o"] = mat(sd[x + "o"])
            else:
                a, r = m["left"], m["right"]
                xl, xr = x + "left.", x + "right."
                qkv = torch.cat([sd[xl + k].float() for k in "qkv"])
                rest = torch.cat([sd[xr + k].float() for k in ("r", "k", "v", "g", "a", "w1")])
                w[x + "in"] = mat(pad16(torch.cat([qkv, rest])))
                bias = torch.cat([sd[xl + k + ".b"].float() if (xl + k + ".b") in sd else torch.zeros(sd[xl + k].shape[0])
                                  for k in "qkv"])
                w[x + "in.b"] = mat(torch.cat([bias, torch.zeros(w[x + "in"].shape[0] - bias.numel())]))
                if a["conv"]:
                    w[xl + "conv"] = f32(torch.cat([sd[xl + k + ".conv"].float() for k in "qkv"]))
                if (xl + "temp") in sd:
                    w[xl + "temp"] = f32(sd[xl + "temp"])
                w[xr + "w2"], w[xr + "w0"], w[xr + "a.b"] = mat(sd[xr + "w2"]), f32(sd[xr + "w0"]), f32(sd[xr + "a.b"])
                # the branch scale of the right branch rides on its norm weight (fp32); the left one on the attention
                # kernel's output scale
                w[xr + "norm"] = f32(sd[xr + "norm"].float() * float(m["right_scale"]))
                w[x + "o"] = mat(torch.cat([sd[xl + "o"].float(), sd[xr + "o"].float()], 1))
            ml = l.get("mlp")
            if ml is not None:
                w[p + "norm2"] = f32(1 + sd[p + "norm2"].float())
                q = p + "mlp."
                E, F_ = ml["router"]["experts"], ml["expert"]["ff"]
                # router rows padded to the GEMM's 16-column grid: the logits come out of the MFMA kernel in fp32
                w[q + "router"] = mat(pad16(sd[q + "router"]))
                if (q + "correction") in sd:
                    w[q + "correction"] = f32(sd[q + "correction"])
                Fp = F_ + (-F_) % (64 if dt == torch.bfloat16 else 16)
                zr = lambda t: torch.cat([t.float(), torch.zeros(Fp - F_, D)])  # noqa: E731
                w[q + "gate_up"] = mat(torch.stack([ops.interleave_gate_up(zr(sd[q + f"e{e}.gate"]), zr(sd[q + f"e{e}.up"]))
                                                    for e in range(E)]))
                w[q + "down"] = mat(torch.stack([torch.cat([sd[q + f"e{e}.down"].float(), torch.zeros(D, Fp - F_)], 1)
                                                 for e in range(E)]))
                if ml.get("shared"):
                    rows = [sd[q + "shared.gate"].float(), sd[q + "shared.up"].float()]
                    if (q + "shared.sg") in sd:
                        rows.append(sd[q + "shared.sg"].float().reshape(1, D))
                    w[q + "shared.in"] = mat(pad16(torch.cat(rows)))
                    w[q + "shared.down"] = mat(sd[q + "shared.down"])
                    if len(rows) == 3:
                        self.shared_gated.add(i)
            if c.side_dim:
                w[p + "side.gate"] = mat(pad16(sd[p + "side.gate"]))
                w[p + "side.proj"], w[p + "side.norm"] = mat(sd[p + "side.proj"]), f32(sd[p + "side.norm"])
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
        c, D = self.cfg, self.cfg.hidden_size
        self.pool.clear()
        self.state = {}
        for i, l in enumerate(c.layers):
            m, tag = l["mixer"], f"l{i}."
            st = dict(shift=self.pool.add(tag + "shift", (1, D)))
            if l["type"] == "gla":
                st["S"] = self.pool.add(tag + "S", (m["heads"], m["dim"], m["vdim"]))
            else:
                a, r = m["left"], m["right"]
                C = (a["heads"] + a["kv_heads"]) * a["dim"] + a["kv_heads"] * a["vdim"]
                if a["conv"] > 1:
                    st["conv"] = self.pool.add(tag + "conv", (a["conv"] - 1, C))
                st["S"] = self.pool.add(tag + "S", (r["heads"], r["dim"], r["dim"]))
            self.state[i] = st

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
    def _gla(self, h, i, seq):
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        H, dk, dv = m["heads"], m["dim"], m["vdim"]
        proj = ops.linear(h, w[x + "in"])
        c1, c2, c3 = H * dk, 2 * H * dk, 2 * H * dk + H * dv
        c4 = c3 + H * dv
        lr = w[x + "a2"].shape[1]
        z = ops.linear(proj[:, c4:c4 + lr], w[x + "a2"], out_dtype=torch.float32)
        alpha = ops.decay_gate(z, w[x + "a2.b"], "sigmoid_root", float(m["tau"]))
        o = ops.dplr_scan(proj[:, :c1], proj[:, c1:c2], proj[:, c2:c3], alpha, None, None, self.state[i]["S"], seq["cu"],
                          seq["slots"], q_scale=dk ** -0.5)
        y = ops.head_norm_gate(o, proj[:, c3:c4], w[x + "norm"], "silu", self.cfg.rms_eps, self.dtype)
        return ops.linear(y, w[x + "o"])

    def _parallel(self, h, i, fb, kv, seq):
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        a, r = m["left"], m["right"]
        H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        Hr, d = r["heads"], r["dim"]
        xl, xr = x + "left.", x + "right."
        st = self.state[i]
        proj = ops.linear(h, w[x + "in"], w[x + "in.b"])
        T = h.shape[0]
        cq, ck = H * dk, (H + G) * dk
        C = ck + G * dv
        both = torch.empty(T, H * dv + Hr * d, dtype=self.dtype, device=h.device)
        # left: chunk-local attention over the paged cache
        qkv = proj[:, :C]
        if a["conv"]:
            cs = st.get("conv")
            if cs is None:  # one tap: a scale per channel, nothing to remember
                cs = torch.zeros(self.pool.n_slots + 1, 0, C, dtype=torch.float32, device=h.device)
            y = ops.conv_silu(qkv, w[xl + "conv"], cs, seq["cu"], seq["slots"], act=False)
            if "conv" in st:
                ops.state_tail_write(qkv, st["conv"], seq["cu"], seq["slots"])
            qkv = y
        kc, vc = kv.layer(self.kv_index[i])
        q = ops.rotary_kv_write(qkv[:, :cq], qkv[:, cq:ck], qkv[:, ck:], fb.positions, fb.slots, kc, vc, H, G, dk, dv,
                                int(a["rot"]["dims"]), float(a["rot"]["base"]))
        ops.window_attention(q, kc, vc, seq["bt"], seq["cu"], seq["ctx"], H, G, dk, dv, float(a["scale"]),
                             chunk=int((a.get("mask") or {}).get("size") or 0), head_scale=w.get(xl + "temp"),
                             sink=SINK_SCORE, out=both[:, : H * dv], out_scale=float(m["left_scale"]))
        # right: generalised delta rule
        n = Hr * d
        c0 = C
        rr, rk, rv, rg, ra = (proj[:, c0 + j * n:c0 + (j + 1) * n] for j in range(5))
        lr = w[xr + "w2"].shape[1]
        lw = ops.act_mul(proj[:, c0 + 5 * n:c0 + 5 * n + lr], None, "tanh_cap", self.dtype, cap=1.0)
        decay = ops.decay_gate(ops.linear(lw, w[xr + "w2"], out_dtype=torch.float32), w[xr + "w0"], "exp_sigmoid",
                               DECAY_RATE)
        av, bv = ops.unit_key_removal(rk, ra, w[xr + "a.b"], Hr, d, UNIT_EPS)
        o = ops.dplr_scan(rr, rk, rv, decay, av, bv, st["S"], seq["cu"], seq["slots"])
        ops.head_norm_gate(o, rg, w[xr + "norm"], "sigmoid", self.cfg.rms_eps, self.dtype, out=both[:, H * dv:])
        return ops.linear(both, w[x + "o"])

    # ------------------------------------------------------------------ feed-forward
    def _moe(self, h, i):
        ml, w, q = self.cfg.layers[i]["mlp"], self.w, f"l{i}.mlp."
        r = ml["router"]
        E, top = r["experts"], r["top"]
        logits = ops.linear(h, w[q + "router"], out_dtype=torch.float32)[:, :E]
        g = r["groups"]
        ids, wts = ops.moe_route(logits, top, score="sigmoid", bias=w.get(q + "correction"), eps=ROUTE_EPS,
                                 groups=(g["count"], g["keep"]), scale=float(r["scale"]))
        shared = sgate = None
        if ml.get("shared"):
            Fs = w[q + "shared.down"].shape[1]
            gu = ops.linear(h, w[q + "shared.in"])
            mid = ops.act_mul(gu[:, :Fs], gu[:, Fs:2 * Fs], "clamp_glu", self.dtype, cap=float(ml["shared"]["limit"]))
            shared = ops.linear(mid, w[q + "shared.down"])
            sgate = gu[:, 2 * Fs:2 * Fs + 1] if i in self.shared_gated else None
        _rows, offs, pos = ops.moe_dispatch(ids, E)
        n = h.shape[0] * top
        mid = ops.moe_gemm(h, _rows, w[q + "gate_up"], offs, n, act="clamp_glu", act_param=float(ml["expert"]["limit"]))
        dn = ops.moe_gemm(mid, None, w[q + "down"], offs, n)
        return ops.moe_combine(dn, pos, wts, shared, residual_gate=sgate)

    # ------------------------------------------------------------------ forward
    def forward(self, fb: ForwardBatch, kv, decode_ws=None) -> torch.Tensor:
        """Returns fp32 logits [len(sample_rows), vocab]."""
        c, w, dt = self.cfg, self.w, self.dtype
        if fb.extra is None:  # direct forward without the engine hook
            self.prepare_batch(fb)
        seq = dict(fb.extra)
        if "ctx" not in seq:  # captured decode graph: one row per sequence, the engine's static ctx / page tables
            seq["ctx"], seq["bt"] = fb.decode_ctx, fb.decode_block_tables
        eps, L, sdim = c.rms_eps, len(c.layers), c.side_dim
        res = ops.embed_scale_f32(fb.token_ids, w["embed"], 1.0)
        side = ops.embed_scale_f32(fb.token_ids, w["side.embed"], 1.0) if sdim else None
        h = ops.add_rmsnorm_f32(res, None, 1.0, w["l0.norm1"], eps, dt) if L else None
        for i, l in enumerate(c.layers):
            p = f"l{i}."
            st = self.state[i]
            if (p + "shift") in w:
                hs = ops.token_shift_mix(h, w[p + "shift"], st["shift"].view(-1, h.shape[1]), seq["cu"], seq["slots"])[0]
                ops.state_tail_write(h, st["shift"], seq["cu"], seq["slots"])
                h = hs
            pend = self._gla(h, i, seq) if l["type"] == "gla" else self._parallel(h, i, fb, kv, seq)
            if l.get("mlp") is not None:
                h = ops.add_rmsnorm_f32(res, pend, 1.0, w[p + "norm2"], eps, dt)
                pend = self._moe(h, i)
            last = i + 1 == L
            nxt = None if last else w[f"l{i + 1}.norm1"]
            if sdim:
                xb = ops.add_rmsnorm_f32(res, pend, 1.0, None, eps, dt)
                g = ops.linear(xb, w[p + "side.gate"], out_dtype=torch.float32)[:, :sdim]
                g = ops.act_mul(g, side[:, i * sdim:(i + 1) * sdim], "gelu_tanh", dt)
                y = ops.linear(g, w[p + "side.proj"], out_dtype=torch.float32)
                h = ops.gated_norm_add_f32(res, y, None, w[p + "side.norm"], eps, nxt, None if last else dt)
            else:
                h = ops.add_rmsnorm_f32(res, pend, 1.0, nxt, eps, None if last else dt)
            if self.capture_residuals is not None:
                self.capture_residuals.append(res.clone())
        if fb.sample_rows is not None:
            res = res.index_select(0, fb.sample_rows)
        xf = ops.add_rmsnorm_f32(res, None, 1.0, w["final.norm"], eps, dt)
        return ops.linear(xf, w["head"], out_dtype=torch.float32)[:, : c.vocab_size]
