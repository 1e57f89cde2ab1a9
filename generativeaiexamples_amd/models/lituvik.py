"""Lituvik: a hybrid decoder whose layer list mixes latent attention, constant-decay linear attention and selective
state-space layers, with statistics-free tanh norms, an optional looped block and dense or mixture-of-experts
feed-forwards.

Architecture (every size and constant comes from ``config.json``; the layer list may hold the mixers in any order):
  * token embedding; the output head is its own matrix; logits are capped by ``cap * tanh(logits / cap)``;
  * a layer is pre-norm: ``x += mixer(N1(x))`` then ``x += ff(N2(x))``; every norm is a dynamic tanh
    ``tanh(alpha x) * w + b`` (no mean, no variance); a layer may have no feed-forward;
  * ``loop``: layers start .. stop - 1 run ``times`` passes with the same weights, every pass with its own cache /
    state; before every pass but the first the embedding output is added to the stream;
  * mixer ``latent_attention``: per token one low-rank latent ``c = rmsnorm(W_dkv h)[:kv_rank]`` and one rotated key
    part shared by all heads; keys and values of a head are linear maps of c. Queries are [dim plain | rot_dim
    rotated] per head; rotation with the "rotate half" pairing, frequencies stretched by a wavelength-dependent ramp
    (``rot.scaling``) and cos / sin scaled by ``0.1 ln(factor) + 1``; sliding window; softmax;
  * mixer ``lightning``: linear attention ``S <- decay_h S + k v^T, o = S^T q`` on silu(q), silu(k), silu(v), a
    whole-row RMS norm, a sigmoid gate;
  * mixer ``mamba1``: [x | z] projection, short causal convolution + SiLU on x, input-dependent step size, B and C,
    ``S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n``, ``y = S C + D x``, times silu(z);
  * feed-forward ``dense``: ``W_down relu(W_up h)^2``; ``moe``: softmax router over experts + identity experts, the
    choice made with an additive correction, weights = chosen scores renormalised, experts ``W_down (silu(W_gate h) *
    W_up h)``, identity experts return their input, plus an always-on shared expert.

MI355X mapping. The residual stream, norms, positions and angles, attention scores and weights, router, decays, step
sizes and recurrent states are fp32; projections run in the model dtype (bf16 MFMA GEMMs with fp32 accumulation, or
true fp32). Latent attention never expands keys or values: the paged cache holds ONE row [c | rotated key] per token
(one kv head), the query is folded through the key expansion (``q_plain W_uk``) so scores are taken against the cached
row directly, the weighted sum runs over c and is expanded through ``W_uv`` afterwards - the cache is (kv_rank + rot_dim)
elements per token instead of heads x (dim + rot_dim + vdim), and the attention kernels are the engine's paged window
kernels with one kv head. Recurrent states (linear-attention matrices, state-space states, convolution tails) live in
the engine's state slot pool. A step's rows - prompt portions and single decoded tokens alike - go through the same HIP
kernels, addressed by device-side (cu, slot, ctx) vectors, so pure-decode steps replay a captured HIP graph.
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

MIXERS = ("latent_attention", "lightning", "mamba1")
ROUTE_EPS = 1e-20      # added to the sum of the chosen router scores


@dataclass
class LituvikConfig:
    vocab_size: int
    hidden_size: int
    layers: Tuple[dict, ...]                 # {"type", "mixer": {...}, "mlp": {"kind": "dense" | "moe", ...} | None}
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0                      # 0: no looped block
    rms_eps: float = 1e-6
    logit_softcap: float = 0.0               # 0: logits are not capped
    name: str = "lituvik"
    max_position: int = 1 << 20              # angles are computed from the position: no table to outgrow
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()

    def __post_init__(self):
        layers = []
        for i, l in enumerate(self.layers):
            if l["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
            m = dict(l["mixer"])
            if l["type"] == "latent_attention":
                m.setdefault("vdim", m["dim"])
                m.setdefault("rot_dim", 0)
                m.setdefault("scale", (m["dim"] + m["rot_dim"]) ** -0.5)
                rot = dict(m.get("rot") or {})
                rot.setdefault("base", 10000.0)
                dims = int(rot.setdefault("dims", m["rot_dim"]))
                if dims % 2 or not 0 <= dims <= m["rot_dim"]:
                    raise ValueError(f"layer {i}: the rotation covers an even number of the rot_dim channels")
                m["rot"] = rot
            elif l["type"] == "lightning":
                m.setdefault("vdim", m["dim"])
                if len(m["decay"]) != m["heads"]:
                    raise ValueError(f"layer {i}: one decay per head")
            else:
                m.setdefault("conv", 4)
                m.setdefault("dt_rank", max(1, self.hidden_size // 16))
            ml = l.get("mlp")
            if ml is not None:
                ml = dict(ml)
                kind = ml.setdefault("kind", "dense")
                if kind not in ("dense", "moe"):
                    raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
                if kind == "moe":
                    r = dict(ml["router"])
                    r.setdefault("identity", 0)
                    if not 1 <= r["top"] <= min(16, r["experts"] + r["identity"]):
                        raise ValueError(f"layer {i}: 1 <= top <= min(16, experts + identity)")
                    ml["router"] = r
            layers.append(dict(l, mixer=m, mlp=ml))
        self.layers = tuple(layers)
        if self.loop_times and not (0 <= self.loop_start < self.loop_stop <= len(self.layers)):
            raise ValueError("loop: need 0 <= start < stop <= number of layers")

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def head_dim(self) -> int:  # engine sizing hooks: the widest cached key row
        return max([l["mixer"]["kv_rank"] + l["mixer"]["rot_dim"] for l in self.layers
                    if l["type"] == "latent_attention"] or [16])

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
    def from_json(path_or_dict) -> "LituvikConfig":
        if isinstance(path_or_dict, dict):
            c, name = path_or_dict, "lituvik"
        else:
            with open(os.path.join(path_or_dict, "config.json")) as f:
                c = json.load(f)
            name = os.path.basename(os.path.normpath(path_or_dict)) or "lituvik"
        lp = c.get("loop") or {}
        eos = c.get("eos_token_id", ())
        return LituvikConfig(
            vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(c["layers"]),
            loop_start=int(lp.get("start", 0)), loop_stop=int(lp.get("stop", 0)), loop_times=int(lp.get("times", 0)),
            rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)), logit_softcap=float(c.get("logit_softcap") or 0.0),
            name=c.get("name", name), max_position=int(c.get("max_position", 1 << 20)),
            bos_token_id=c.get("bos_token_id"), eos_token_ids=tuple(eos) if isinstance(eos, (list, tuple)) else (eos,))

    @staticmethod
    def tiny(**kw) -> "LituvikConfig":
        att = dict(heads=2, dim=16, rot_dim=8, vdim=24, kv_rank=40, scale=0.2, mask=dict(size=20),
                   rot=dict(base=10000.0, dims=8, scaling=dict(factor=8.0, original=64, fast=16.0, slow=2.0)))
        lin = dict(heads=2, dim=16, vdim=32, decay=[0.8, 0.97])
        ssm = dict(inner=96, state=8, dt_rank=6, conv=3)
        dense = dict(kind="dense", ff=128)
        moe = dict(kind="moe", expert=dict(ff=48), router=dict(experts=5, identity=2, top=3), shared=dict(ff=32))
        base = dict(vocab_size=512, hidden_size=64, name="tiny-lituvik", rms_eps=1e-5, logit_softcap=20.0,
                    loop_start=1, loop_stop=3, loop_times=2,
                    layers=(dict(type="lightning", mixer=lin, mlp=dense), dict(type="latent_attention", mixer=att, mlp=moe),
                            dict(type="mamba1", mixer=ssm, mlp=None), dict(type="latent_attention", mixer=att, mlp=dense)))
        base.update(kw)
        return LituvikConfig(**base)

    @staticmethod
    def sized(width: int, n_layers: int, ff: int, heads: int, head_dim: int, window: int = 1024, vocab: int = 32768,
              experts: int = 8, top: int = 2, pattern: Tuple[str, ...] = MIXERS, **kw) -> "LituvikConfig":
        """A regular stack for benchmarks: `pattern` repeated over n_layers; attention layers carry the experts (two
        active experts of ff / 2 each plus nothing shared would equal a dense ff: here top experts of ff / top)."""
        rot = head_dim // 2
        mix = dict(latent_attention=dict(heads=heads, dim=head_dim, rot_dim=rot, vdim=head_dim, kv_rank=head_dim,
                                         scale=(head_dim + rot) ** -0.5, mask=dict(size=window),
                                         rot=dict(base=10000.0, dims=rot,
                                                  scaling=dict(factor=8.0, original=2048, fast=16.0, slow=2.0))),
                   lightning=dict(heads=heads, dim=head_dim, vdim=head_dim,
                                  decay=[1.0 - 2.0 ** (-5.0 - 3.0 * h / max(1, heads - 1)) for h in range(heads)]),
                   mamba1=dict(inner=2 * width, state=16, dt_rank=max(16, width // 16), conv=4))
        dense = dict(kind="dense", ff=ff)
        moe = dict(kind="moe", expert=dict(ff=ff // top), router=dict(experts=experts, identity=0, top=top))
        layers = tuple(dict(type=pattern[i % len(pattern)], mixer=mix[pattern[i % len(pattern)]],
                            mlp=moe if experts and pattern[i % len(pattern)] == "latent_attention" else dense)
                       for i in range(n_layers))
        base = dict(vocab_size=vocab, hidden_size=width, layers=layers, logit_softcap=30.0,
                    name=f"lituvik-{width}x{n_layers}")
        base.update(kw)
        return LituvikConfig(**base)


def random_state(cfg: LituvikConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """A random checkpoint (tensor names and shapes of the safetensors layout, fp32 values) with magnitudes that keep
    activations, decays and states in a trained model's range."""
    g = torch.Generator().manual_seed(seed)
    D = cfg.hidden_size
    rn = lambda *s, std=1.0: torch.randn(*s, generator=g) * std  # noqa: E731
    un = lambda *s, lo=0.0, hi=1.0: torch.rand(*s, generator=g) * (hi - lo) + lo  # noqa: E731
    lin = lambda o, i: rn(o, i, std=i ** -0.5)  # noqa: E731

    def norm(name):
        sd[name], sd[name + ".b"] = 1 + rn(D, std=0.1), rn(D, std=0.05)
        sd[name + ".alpha"] = un(1, lo=0.3, hi=0.8).reshape(())

    def gated(p, F_):
        sd[p + "gate"], sd[p + "up"], sd[p + "down"] = lin(F_, D) * 1.5, lin(F_, D), lin(D, F_)

    sd: Dict[str, torch.Tensor] = {"embed": rn(cfg.vocab_size, D), "head": lin(cfg.vocab_size, D) * 2.0}
    norm("final.norm")
    for i, l in enumerate(cfg.layers):
        p, m, x = f"l{i}.", l["mixer"], f"l{i}.mix."
        norm(p + "norm1")
        if l["type"] == "latent_attention":
            H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            sd[x + "q"], sd[x + "dkv"] = lin(H * (dn + dr), D) * 2.0, lin(R + dr, D) * 2.0
            sd[x + "dkv.norm"] = 1 + rn(R, std=0.1)
            sd[x + "uk"], sd[x + "uv"] = lin(H * dn, R) * 1.5, lin(H * dv, R)
            sd[x + "o"] = lin(D, H * dv)
        elif l["type"] == "lightning":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            sd[x + "q"], sd[x + "k"], sd[x + "v"] = lin(H * dk, D), lin(H * dk, D), lin(H * dv, D)
            sd[x + "g"], sd[x + "o"] = lin(H * dv, D), lin(D, H * dv)
            sd[x + "norm"] = 1 + rn(H * dv, std=0.1)
        else:
            I, N, rk, K = m["inner"], m["state"], m["dt_rank"], m["conv"]
            sd[x + "in"] = lin(2 * I, D)
            sd[x + "conv"], sd[x + "conv.b"] = rn(I, K, std=K ** -0.5), rn(I, std=0.1)
            sd[x + "x"] = lin(rk + 2 * N, I)
            sd[x + "dt"], sd[x + "dt.b"] = lin(I, rk), un(I, lo=-4.0, hi=-1.0)
            sd[x + "A_log"] = torch.log(un(I, N, lo=0.2, hi=4.0))
            sd[x + "D"] = 1 + rn(I, std=0.2)
            sd[x + "o"] = lin(D, I)
        ml = l.get("mlp")
        if ml is None:
            continue
        norm(p + "norm2")
        if ml["kind"] == "dense":
            sd[p + "mlp.up"], sd[p + "mlp.down"] = lin(ml["ff"], D), lin(D, ml["ff"])
        else:
            r = ml["router"]
            for e in range(r["experts"]):
                gated(p + f"mlp.e{e}.", ml["expert"]["ff"])
            sd[p + "mlp.router"] = lin(r["experts"] + r["identity"], D) * 2.0
            sd[p + "mlp.correction"] = rn(r["experts"] + r["identity"], std=0.05)
            if ml.get("shared"):
                gated(p + "mlp.shared.", ml["shared"]["ff"])
    return sd


class LituvikModel:
    """Weights (plain tensors) + forward for the serving engine (the hooks of LlamaModel / PinavikModel)."""

    has_recurrent_state = True       # no prefix-cache reuse: a cached prefix has no recurrent state to resume from
    attention_backend = "window"     # the paged window attention kernels: no flash-attention tile lists

    def __init__(self, cfg: LituvikConfig, device=None, dtype=torch.bfloat16, dist_ctx: DistContext | None = None,
                 state_slots: Optional[int] = None):
        self.cfg = cfg
        self.ctx = dist_ctx or get_context()
        assert self.ctx.tp_size == 1, "Lituvik runs TP=1"
        self.device = torch.device(device) if device is not None else self.ctx.device
        self.dtype = dtype
        self.runs = cfg.runs()
        att = [r for r in self.runs if cfg.layers[r[0]]["type"] == "latent_attention"]
        self.kv_index = {r: j for j, r in enumerate(att)}
        self.num_kv_layers = len(att)
        self.hq = max([cfg.layers[i]["mixer"]["heads"] for i, _ in att] or [1])
        self.hkv = 1
        self.vocab_local, self.vstart = cfg.vocab_size, 0
        self.lora_names: list = []
        self.w: Dict[str, torch.Tensor] = {}
        self.alpha: Dict[str, float] = {}
        self.rot: Dict[int, Tuple[torch.Tensor, float]] = {}
        self.pool = StatePool(state_slots or int(os.environ.get("GAI_LINEAR_STATE_SLOTS", "64")), self.device)
        self.state: Dict[Tuple[int, int], Dict[str, torch.Tensor]] = {}
        self.capture_residuals: Optional[list] = None  # numerics debugging: the residual stream after every layer run
        self._i32 = dict(dtype=torch.int32, device=self.device)

    # ------------------------------------------------------------------ engine sizing hooks
    def kv_layout(self) -> List[Tuple[int, int, int]]:
        """(kv heads, key size, value size) of every paged cache layer: one per latent-attention layer run, ONE kv
        head whose key row is [latent | rotated key part] and whose value row is the latent."""
        out = []
        for (i, _t) in sorted(self.kv_index, key=self.kv_index.get):
            m = self.cfg.layers[i]["mixer"]
            out.append((1, m["kv_rank"] + m["rot_dim"], m["kv_rank"]))
        return out

    # ------------------------------------------------------------------ weights
    def _fused_ok(self, F_: int) -> bool:
        """The SwiGLU-epilogue GEMM takes bf16 with K % 64 == 0 and interleaved gate / up blocks of 16 rows."""
        return self.dtype == torch.bfloat16 and self.cfg.hidden_size % 64 == 0 and F_ % 16 == 0 \
            and self.device.type == "cuda"

    def load_state(self, sd: Dict[str, torch.Tensor]):
        """Checkpoint tensors (the safetensors names) -> device weights: projections in the model dtype, per-channel
        tables fp32, same-input projections fused, expert matrices stacked (rows padded with zeros to the grouped
        GEMM's grid: a zero gate / up row contributes nothing)."""
        c, dev, dt = self.cfg, self.device, self.dtype
        f32 = lambda t: t.to(torch.float32).to(dev).contiguous()  # noqa: E731
        mat = lambda t: t.to(torch.float32).to(dev, dt).contiguous()  # noqa: E731
        D = c.hidden_size
        w = self.w = {}
        self.alpha, self.rot = {}, {}

        def norm(name):
            w[name], w[name + ".b"] = f32(sd[name]), f32(sd[name + ".b"])
            self.alpha[name] = float(sd[name + ".alpha"].float())

        def gate_up(g, u):
            g, u = g.float(), u.float()
            return mat(ops.interleave_gate_up(g, u) if self._fused_ok(g.shape[0]) else torch.cat([g, u]))

        w["embed"], w["head"] = mat(sd["embed"]), mat(sd["head"])
        norm("final.norm")
        for i, l in enumerate(c.layers):
            p, x, m = f"l{i}.", f"l{i}.mix.", l["mixer"]
            norm(p + "norm1")
            if l["type"] == "latent_attention":
                H, dn, R = m["heads"], m["dim"], m["kv_rank"]
                w[x + "in"] = mat(torch.cat([sd[x + "q"], sd[x + "dkv"]]))
                w[x + "dkv.norm"] = f32(sd[x + "dkv.norm"])
                w[x + "uk"] = mat(sd[x + "uk"].float().reshape(H, dn, R))                     # q_plain [H, T, dn] @ this
                w[x + "uv"] = mat(sd[x + "uv"].float().reshape(H, m["vdim"], R).transpose(1, 2))  # [H, R, dv]
                inv, mag = ops.yarn_inv_freq(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling")) \
                    if m["rot"]["dims"] else (torch.zeros(0), 1.0)
                self.rot[i] = (inv.to(dev), mag)
            elif l["type"] == "lightning":
                w[x + "in"] = mat(torch.cat([sd[x + k] for k in ("q", "k", "v", "g")]))
                w[x + "norm"] = f32(sd[x + "norm"])
                w[x + "decay"] = f32(torch.tensor([float(d) for d in m["decay"]]))
            else:
                w[x + "in"], w[x + "x"], w[x + "dt"] = mat(sd[x + "in"]), mat(sd[x + "x"]), mat(sd[x + "dt"])
                w[x + "conv"], w[x + "conv.b"] = f32(sd[x + "conv"]), f32(sd[x + "conv.b"])
                w[x + "dt.b"], w[x + "D"] = f32(sd[x + "dt.b"]), f32(sd[x + "D"])
                w[x + "A"] = -torch.exp(f32(sd[x + "A_log"]))
            w[x + "o"] = mat(sd[x + "o"])
            ml = l.get("mlp")
            if ml is None:
                continue
            norm(p + "norm2")
            q = p + "mlp."
            if ml["kind"] == "dense":
                w[q + "up"], w[q + "down"] = mat(sd[q + "up"]), mat(sd[q + "down"])
                continue
            r = ml["router"]
            E, F_ = r["experts"], ml["expert"]["ff"]
            # router rows padded to the GEMM's 16-column grid: the logits come out of the MFMA kernel in fp32
            pad = (-(E + r["identity"])) % 16
            w[q + "router"] = mat(torch.cat([sd[q + "router"].float(), torch.zeros(pad, D)]))
            w[q + "correction"] = f32(sd[q + "correction"])
            if E:
                Fp = F_ + (-F_) % (64 if dt == torch.bfloat16 else 16)
                zr = lambda t: torch.cat([t.float(), torch.zeros(Fp - F_, D)])  # noqa: E731
                w[q + "gate_up"] = mat(torch.stack([ops.interleave_gate_up(zr(sd[q + f"e{e}.gate"]), zr(sd[q + f"e{e}.up"]))
                                                    for e in range(E)]))
                w[q + "down"] = mat(torch.stack([torch.cat([sd[q + f"e{e}.down"].float(), torch.zeros(D, Fp - F_)], 1)
                                                 for e in range(E)]))
            if ml.get("shared"):
                w[q + "shared.gate_up"] = gate_up(sd[q + "shared.gate"], sd[q + "shared.up"])
                w[q + "shared.down"] = mat(sd[q + "shared.down"])
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
            if l["type"] == "lightning":
                self.state[r] = dict(S=self.pool.add(tag + "S", (m["heads"], m["dim"], m["vdim"])))
            elif l["type"] == "mamba1":
                self.state[r] = dict(conv=self.pool.add(tag + "conv", (m["conv"] - 1, m["inner"])),
                                     S=self.pool.add(tag + "S", (m["inner"], m["state"])))

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
    def _latent_attention(self, h, i, run, fb, kv, seq):
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        T = h.shape[0]
        proj = ops.linear(h, w[x + "in"])
        nq = H * (dn + dr)
        q = proj[:, :nq]
        # the plain query part folded through the key expansion: scores against the cached latent need no keys
        qcat = torch.empty(T, H, R + dr, dtype=self.dtype, device=h.device)
        qcat[:, :, :R] = torch.bmm(q.view(T, H, dn + dr)[:, :, :dn].transpose(0, 1), w[x + "uk"]).transpose(0, 1)
        kc, vc = kv.layer(self.kv_index[run])
        inv, mag = self.rot[i]
        ops.latent_kv_write(q, proj[:, nq:], w[x + "dkv.norm"], inv, mag, fb.positions, fb.slots, qcat.view(T, -1), kc,
                            vc, H, dn, dr, R, self.cfg.rms_eps)
        lat = ops.window_attention(qcat.view(T, -1), kc, vc, seq["bt"], seq["cu"], seq["ctx"], H, 1, R + dr, R,
                                   float(m["scale"]), 0.0, int((m.get("mask") or {}).get("size") or 0))
        # the weighted latents expanded to the heads' values
        val = torch.bmm(lat.view(T, H, R).transpose(0, 1), w[x + "uv"]).transpose(0, 1).reshape(T, H * dv)
        return ops.linear(val, w[x + "o"])

    def _lightning(self, h, i, run, seq):
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        H, dk, dv = m["heads"], m["dim"], m["vdim"]
        proj = ops.linear(h, w[x + "in"])
        n = 2 * H * dk + H * dv
        qkv = ops.act_mul(proj[:, :n], None, "silu", torch.float32)
        o = ops.linear_attention_scan(qkv[:, :H * dk], qkv[:, H * dk:2 * H * dk], qkv[:, 2 * H * dk:], w[x + "decay"],
                                      self.state[run]["S"], seq["cu"], seq["slots"])
        y = ops.head_norm_gate(o.view(-1, 1, H * dv), proj[:, n:], w[x + "norm"], "sigmoid", self.cfg.rms_eps, self.dtype)
        return ops.linear(y, w[x + "o"])

    def _mamba1(self, h, i, run, seq):
        m, w, x = self.cfg.layers[i]["mixer"], self.w, f"l{i}.mix."
        I, N, rk = m["inner"], m["state"], m["dt_rank"]
        st = self.state[run]
        proj = ops.linear(h, w[x + "in"])
        xin = proj[:, :I]
        xc = ops.conv_silu(xin, w[x + "conv"], st["conv"], seq["cu"], seq["slots"], bias=w[x + "conv.b"], act=True)
        ops.state_tail_write(xin, st["conv"], seq["cu"], seq["slots"])
        low = ops.linear(xc if self.dtype == torch.float32 else xc.to(self.dtype), w[x + "x"])
        dt = ops.linear(low[:, :rk], w[x + "dt"], out_dtype=torch.float32)
        y = ops.selective_scan(xc, dt, w[x + "dt.b"], w[x + "A"], low[:, rk:rk + N], low[:, rk + N:], w[x + "D"],
                               proj[:, I:], st["S"], seq["cu"], seq["slots"], self.dtype)
        return ops.linear(y, w[x + "o"])

    # ------------------------------------------------------------------ feed-forwards
    def _gated(self, h, wgu, wdown):
        """W_down (silu(W_gate h) * W_up h): one GEMM with the gate in its epilogue where the shape allows it."""
        F_ = wdown.shape[1]
        if self._fused_ok(F_):
            return ops.linear(ops.linear(h, wgu, act="swiglu"), wdown)
        gu = ops.linear(h, wgu)
        return ops.linear(ops.act_mul(gu[:, :F_], gu[:, F_:], "silu"), wdown)

    def _moe(self, h, i):
        ml, w, q = self.cfg.layers[i]["mlp"], self.w, f"l{i}.mlp."
        r = ml["router"]
        E, NI, top = r["experts"], r["identity"], r["top"]
        logits = ops.linear(h, w[q + "router"], out_dtype=torch.float32)[:, :E + NI]
        ids, wts = ops.moe_route(logits, top, renorm=True, bias=w[q + "correction"], eps=ROUTE_EPS)
        shared = self._gated(h, w[q + "shared.gate_up"], w[q + "shared.down"]) if ml.get("shared") else None
        _rows, offs, pos = ops.moe_dispatch(ids, E + NI)
        n = h.shape[0] * top
        if E:
            mid = ops.moe_gemm(h, _rows, w[q + "gate_up"], offs, n, act="swiglu")
            dn = ops.moe_gemm(mid, None, w[q + "down"], offs, n)
        else:
            dn = h.new_zeros(0, h.shape[1])
        return ops.moe_combine(dn, pos, wts, shared, ids=ids if NI else None, n_real=E, identity=h if NI else None)

    # ------------------------------------------------------------------ forward
    def forward(self, fb: ForwardBatch, kv, decode_ws=None) -> torch.Tensor:
        """Returns fp32 logits [len(sample_rows), vocab]."""
        c, w, dt, al = self.cfg, self.w, self.dtype, self.alpha
        if fb.extra is None:  # direct forward without the engine hook
            self.prepare_batch(fb)
        seq = dict(fb.extra)
        if "ctx" not in seq:  # captured decode graph: one row per sequence, the engine's static ctx / page tables
            seq["ctx"], seq["bt"] = fb.decode_ctx, fb.decode_block_tables
        x0 = ops.embed_scale_f32(fb.token_ids, w["embed"], 1.0)
        res = x0.clone() if c.loop_times > 1 else x0
        pend = None
        for (i, t) in self.runs:
            l = c.layers[i]
            p = f"l{i}."
            again = x0 if (t > 0 and i == c.loop_start) else None   # a later pass re-injects the embedding output
            h = ops.add_dyt_f32(res, pend, again, al[p + "norm1"], w[p + "norm1"], w[p + "norm1.b"], dt)
            if l["type"] == "latent_attention":
                pend = self._latent_attention(h, i, (i, t), fb, kv, seq)
            elif l["type"] == "lightning":
                pend = self._lightning(h, i, (i, t), seq)
            else:
                pend = self._mamba1(h, i, (i, t), seq)
            ml = l.get("mlp")
            if ml is not None:
                h = ops.add_dyt_f32(res, pend, None, al[p + "norm2"], w[p + "norm2"], w[p + "norm2.b"], dt)
                if ml["kind"] == "dense":
                    pend = ops.linear(ops.act_mul(ops.linear(h, w[p + "mlp.up"]), None, "relu2"), w[p + "mlp.down"])
                else:
                    pend = self._moe(h, i)
            if self.capture_residuals is not None:
                ops.add_dyt_f32(res, pend, None, 1.0, None, None, None)
                pend = None
                self.capture_residuals.append(res.clone())
        if fb.sample_rows is not None:
            res = res.index_select(0, fb.sample_rows)
            pend = pend.index_select(0, fb.sample_rows) if pend is not None else None
        xf = ops.add_dyt_f32(res, pend, None, al["final.norm"], w["final.norm"], w["final.norm.b"], dt)
        logits = ops.linear(xf, w["head"], out_dtype=torch.float32)[:, : c.vocab_size]
        if c.logit_softcap > 0:
            logits = ops.act_mul(logits, None, "tanh_cap", torch.float32, cap=c.logit_softcap)
        return logits
