"""Prefill and decode throughput of the hybrid decoders at layer sizes of real models (random weights), side by side:
Vipolix (gated linear attention layers and layers of chunk-local attention beside a generalised delta rule, token shift,
group-routed clamped experts plus a gated shared expert on every layer, a per-layer token input; fp32 residual / state),
Lituvik (latent attention over a one-row-per-token cache, constant-decay linear attention, selective state-space scan,
tanh norms, routed experts on the attention layers; fp32 residual / state), Ronavik (sigmoid attention beside a gated linear recurrence, state-space scan layers, sigmoid-routed experts, fp32
post-norm residual / state), Pinavik (windowed attention + WKV + channel-decay delta rule, fp32 residual / state) and
Qwen3-Next (gated full attention + gated DeltaNet), built at the same width, depth, head geometry and active
feed-forward size (Ronavik, and Lituvik's attention layers: 8 experts of half the dense size, 2 per token; the others
dense). `bench.py --hybrid` runs
it; the default workload of bench.py is untouched.

Both models run through the serving engine (native scheduler, paged KV, state slots, decode graphs):
  * prefill: one prompt of T tokens in one step -> tokens / s;
  * decode:  B sequences with a context of C tokens, N single-token steps each -> tokens / s.
"""
from __future__ import annotations

import time

import torch

SIZES = {  # name: (width, layers, ff, heads, head_dim)
    "1k": (1024, 6, 2816, 8, 128),
    "2k": (2048, 6, 5632, 16, 128),
    "4k": (4096, 6, 11008, 32, 128),
}


def add_args(ap):
    ap.add_argument("--hybrid", action="store_true",
                    help="prefill / decode throughput of Vipolix, Lituvik, Ronavik, Pinavik and Qwen3-Next at equal layer sizes "
                         "(one GPU)")
    ap.add_argument("--hybrid-sizes", default="1k,2k", help="comma list of " + ",".join(SIZES))
    ap.add_argument("--hybrid-models", default="vipolix,lituvik,ronavik,pinavik,qwen3-next")
    ap.add_argument("--hybrid-prefill", default="2048,8192", help="prompt lengths of the prefill measurement")
    ap.add_argument("--hybrid-decode", default="1,16,64", help="batch sizes of the decode measurement")
    ap.add_argument("--hybrid-context", type=int, default=1024)
    ap.add_argument("--hybrid-window", type=int, default=1024)


def build(model: str, size: str, window: int, device):
    W, L, F, H, hd = SIZES[size]
    if model == "vipolix":
        from ..models.vipolix import VipolixConfig, VipolixModel

        cfg = VipolixConfig.sized(W, L, F, H, hd, chunk=window, experts=8, top=2)
        return VipolixModel(cfg, device=device).random_init(0)
    if model == "lituvik":
        from ..models.lituvik import LituvikConfig, LituvikModel

        cfg = LituvikConfig.sized(W, L, F, H, hd, window=window, experts=8, top=2)
        return LituvikModel(cfg, device=device).random_init(0)
    if model == "ronavik":
        from ..models.ronavik import RonavikConfig, RonavikModel

        cfg = RonavikConfig.sized(W, L, F // 2, H, hd, experts=8, top=2, max_position=16384)
        return RonavikModel(cfg, device=device).random_init(0)
    if model == "pinavik":
        from ..models.pinavik import PinavikConfig, PinavikModel

        cfg = PinavikConfig.sized(W, L, F, H, hd, window=window)
        return PinavikModel(cfg, device=device).random_init(0)
    from ..models.qwen3_next import Qwen3NextConfig, Qwen3NextModel

    cfg = Qwen3NextConfig(name=f"qwen3-next-{size}", vocab_size=32768, hidden_size=W, intermediate_size=F, num_layers=L,
                          num_heads=H, num_kv_heads=max(1, H // 4), head_dim=hd, linear_num_key_heads=max(1, H // 2),
                          linear_num_value_heads=H, linear_key_head_dim=hd, linear_value_head_dim=hd, num_experts=0,
                          mlp_only_layers=tuple(range(L)), full_attention_interval=3, max_position=32768,
                          bos_token_id=1, eos_token_ids=(2,))
    return Qwen3NextModel(cfg, device=device).random_init(0)


def _engine(model, max_seqs: int, tokens: int):
    from ..engine import EngineConfig, LLMEngine
    from ..engine.tokenizer import small_byte_tokenizer

    return LLMEngine(model, small_byte_tokenizer(512), EngineConfig(
        max_num_seqs=max_seqs, num_blocks=max(64, (tokens + 15) // 16 + max_seqs), max_model_len=16384,
        max_batched_tokens=1 << 20, prefill_chunk=1 << 20, prefix_cache=False, decode_steps=1,
        graph_batch_sizes=(1, 16, 64)))


def _sync():
    if torch.cuda.is_available():
        torch.cuda.synchronize()


def measure(model, prefill_lens, decode_batches, context: int, steps: int, warmup: int) -> dict:
    from ..engine import SamplingParams

    out = {"prefill": {}, "decode": {}}
    g = torch.Generator().manual_seed(0)
    V = model.cfg.vocab_size
    prompt = lambda n: torch.randint(3, V, (n,), generator=g).tolist()  # noqa: E731
    one = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
    for T in prefill_lens:
        eng = _engine(model, 2, T + 64)
        ts = []
        for i in range(warmup + steps):
            p = prompt(T)
            _sync()
            t0 = time.perf_counter()
            eng.generate([p], one)
            _sync()
            if i >= warmup:
                ts.append(time.perf_counter() - t0)
        out["prefill"][T] = dict(tokens_per_s=T * len(ts) / sum(ts), ms=1e3 * sum(ts) / len(ts))
        eng.close()
    for B in decode_batches:
        N = 32
        eng = _engine(model, B, B * (context + N * (warmup + steps) + 32))
        sp = SamplingParams(temperature=0.0, max_tokens=N * (warmup + steps) + 1, ignore_eos=True)
        for _ in range(B):
            eng.add_request(prompt(context), sp)
        while eng.sched.num_waiting() > 0 or eng.stats["decode_tokens"] == 0:
            eng.step()  # prefill, first decode step (captures the graph)
        ts = []
        for i in range(warmup + steps):
            _sync()
            d0, t0 = eng.stats["decode_tokens"], time.perf_counter()
            while eng.stats["decode_tokens"] - d0 < B * N and eng.has_work():
                eng.step()
            _sync()
            if i >= warmup:
                ts.append((eng.stats["decode_tokens"] - d0, time.perf_counter() - t0))
        tok, sec = sum(a for a, _ in ts), sum(b for _, b in ts)
        out["decode"][B] = dict(tokens_per_s=tok / sec, ms_per_step=1e3 * sec / max(1, tok // B))
        eng.close()
    return out


def run(args) -> dict:
    dev = torch.device("cuda", 0) if torch.cuda.is_available() else torch.device("cpu")
    res = {}
    for size in args.hybrid_sizes.split(","):
        for name in args.hybrid_models.split(","):
            model = build(name, size, args.hybrid_window, dev)
            r = measure(model, [int(x) for x in args.hybrid_prefill.split(",") if x],
                        [int(x) for x in args.hybrid_decode.split(",") if x], args.hybrid_context,
                        max(1, args.steps), max(1, args.warmup))
            r["params_m"] = round(model.num_params() / 1e6, 1)
            res[f"{name}-{size}"] = r
            del model
            if dev.type == "cuda":
                torch.cuda.empty_cache()
    return {"metric": "hybrid_decoder_throughput", "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16",
            "data": "synthetic", "steps": args.steps, "warmup": args.warmup, "results": res}
