"""Prefill and decode throughput of Ramalix at layer sizes of a real model, beside Feruzen (the closest existing model: layers
listed one by one, input convolutions with carried tails, delta-rule layers with short convolutions beside softmax attention
over the paged cache, softmax-routed experts with a shared one, the same one-step runtime) at equal width, head counts, head
sizes, expert sizes and layer-run count.  Random weights, bf16, one GPU.
`python bench.py --model ramalix [--rx-size mid]` prints one JSON line; the default bench workload is untouched."""
import json
import time

SIZES = {
    # width; attention heads / kv heads (two maps of 64 -> 128 query values, 128 value values; the block-masked form 128 / 128);
    # delta: value heads / key heads x 128 x 128, ranks of the low-rank pairs; experts x expert ff, top, shared ff; vocab
    "small": dict(width=1024, heads=8, kv=2, lin_v=8, lin_k=4, rank=64, experts=16, eff=512, top=4, sff=1024, vocab=32768),
    "mid": dict(width=2048, heads=16, kv=4, lin_v=16, lin_k=8, rank=96, experts=32, eff=1024, top=4, sff=2048, vocab=65536),
    "large": dict(width=4096, heads=32, kv=8, lin_v=32, lin_k=16, rank=128, experts=32, eff=1536, top=6, sff=3072, vocab=65536),
}
RUNS = 8        # Ramalix: four layers (two-map attention, block attention, channel delta, block attention) walked twice
BLOCK = 256     # positions per block of the block-masked attention


def ramalix_config(s):
    moe = {"kind": "moe", "expert": {"ff": s["eff"]}, "router": {"experts": s["experts"], "top": s["top"], "groups": {"count": 4, "keep": 2}},
           "shared": {"ff": s["sff"]}}
    two = {"heads": s["heads"], "kv_heads": s["kv"], "dim": 64, "vdim": 128, "diff": 0.6, "scale": 0.125,
           "q_temp": {"coef": 0.5, "every": 128}}
    blk = {"heads": s["heads"], "kv_heads": s["kv"], "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "mask": {"size": BLOCK},
           "rot": {"base": 1e6, "dims": 64}}
    dl = {"heads": s["lin_v"], "kv_heads": s["lin_k"], "dim": 128, "vdim": 128, "conv": 4, "a_rank": s["rank"], "g_rank": s["rank"]}
    layers = [{"type": "attention", "mixer": two, "mlp": moe}, {"type": "attention_2", "mixer": blk, "mlp": moe},
              {"type": "channel_delta", "mixer": dl, "mlp": moe}, {"type": "attention_2", "mixer": blk, "mlp": moe}]
    return {"architecture": "Ramalix", "width": s["width"], "vocab": s["vocab"], "norm": {"eps": 1e-5}, "canon": {"taps": 4},
            "residual_mult": 0.7, "logit_scale": 0.5, "loop": {"start": 0, "stop": 4, "times": RUNS // 4}, "layers": layers}


def feruzen_config(s):
    """the same layer runs as eight Feruzen layers: attention layers with 128-wide heads (beside one small matrix memory head,
    which that design's attention layers cannot go without; 128 values wide so that the joint output projection keeps a width
    the tuned GEMM routes take), delta layers of equal heads, the same experts on every layer"""
    moe = {"kind": "moe", "expert": {"ff": s["eff"], "limit": 7.0}, "router": {"experts": s["experts"], "top": s["top"]},
           "shared": {"ff": s["sff"], "limit": 7.0}}
    par = {"left": {"heads": s["heads"], "kv_heads": s["kv"], "dim": 128, "vdim": 128, "rot": {"base": 1e6, "dims": 64}, "scale": 128 ** -0.5},
           "right": {"heads": 1, "dim": 16, "vdim": 128, "gate_cap": 15.0}, "left_scale": 1.0, "right_scale": 1.0}
    dl = {"heads": s["lin_v"], "kv_heads": s["lin_k"], "dim": 128, "vdim": 128, "conv": 4}
    four = [{"type": "parallel", "mixer": par, "mlp": moe}, {"type": "parallel", "mixer": par, "mlp": moe},
            {"type": "delta", "mixer": dl, "mlp": moe}, {"type": "parallel", "mixer": par, "mlp": moe}]
    return {"architecture": "Feruzen", "width": s["width"], "vocab": s["vocab"], "norm": {"eps": 1e-5, "groups": 1},
            "canon": {"taps": 4}, "layers": four * (RUNS // 4)}


def _timed(fn, iters):
    fn()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    return (time.perf_counter() - t0) / iters


def measure(engine_cls, cfg, s, prompt_len, ctx, batches, iters, phase="all"):
    eng = engine_cls(cfg, max_tokens=max(batches) * (ctx + 64) + prompt_len + 64, max_requests=max(batches),
                     dtype="bfloat16").fill_synthetic(seed=1, std=0.02)
    prompt = [(100 + i) % s["vocab"] for i in range(prompt_len)]
    out = {"weight_bytes": eng.weight_bytes(), "state_floats_per_request": eng.state_floats()}

    def prefill():
        r = eng.new_request()
        eng.step([(r, prompt)], logits=False, tokens=True)
        eng.drop_request(r)
    if phase in ("all", "prefill"):
        out["prefill_tok_s"] = round(prompt_len / _timed(prefill, iters), 1)
        out["prefill_device_ms"] = round(eng.last_step_ms(), 3)
    for bs in batches if phase in ("all", "decode") else ():
        rids = [eng.new_request() for _ in range(bs)]
        eng.step([(r, prompt[:ctx]) for r in rids], logits=False, tokens=True)
        dt = _timed(lambda: eng.step([(r, [7]) for r in rids], logits=False, tokens=True), max(iters, 20))
        out["decode_bs%d_tok_s" % bs] = round(bs / dt, 1)
        out["decode_bs%d_device_ms" % bs] = round(eng.last_step_ms(), 3)
        for r in rids:
            eng.drop_request(r)
    eng.close()
    return out


def run(args):
    from .feruzen import FeruzenEngine
    from .ramalix import RamalixEngine
    sizes = [args.rx_size] if args.rx_size != "all" else list(SIZES)
    which = getattr(args, "rx_only", "both")
    phase = getattr(args, "rx_phase", "all")        # one phase alone gives a kernel trace of that phase only
    batches = (1, 4) if phase == "all" else (1,)
    res = {}
    for name in sizes:
        s = SIZES[name]
        res[name] = {"layer_runs": RUNS, "sizes": s}
        if which in ("both", "ramalix"):
            res[name]["ramalix"] = measure(RamalixEngine, ramalix_config(s), s, args.ctx, args.ctx, batches, max(2, args.warmup), phase)
        if which in ("both", "feruzen"):
            res[name]["feruzen_equal_size"] = measure(FeruzenEngine, feruzen_config(s), s, args.ctx, args.ctx, batches, max(2, args.warmup), phase)
    print(json.dumps({"metric": "ramalix_vs_feruzen_layer_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
                      "n_gpus": 1, "prompt_len": args.ctx, "decode_ctx": args.ctx, "results": res}))
    return 0
