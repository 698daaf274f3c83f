"""Prefill and decode throughput of Kukulorn at layer sizes of a real model, beside Feruzen (the closest existing model: layers
listed one by one, short convolutions with carried tails, softmax attention over the paged cache beside a recurrent matrix state
in one mixer, dense gated feed-forwards, the same one-step runtime) at equal width, head counts, head sizes, recurrent state
size, feed-forward size and layer-run count.  Random weights, bf16, one GPU.
`python bench.py --model kukulorn [--kk-size mid]` prints one JSON line; the default bench workload is untouched."""
import json
import time

SIZES = {
    # width; attention heads / kv heads x 128; state-space heads x 64 values x 128 states (Feruzen: memory heads x 128 x 256, the
    # same floats of state and the same inner width); dense ff; vocab
    "small": dict(width=1024, heads=8, kv=2, ssm_heads=16, mm_heads=4, ff=3072, vocab=32768),
    "mid": dict(width=2048, heads=16, kv=4, ssm_heads=32, mm_heads=8, ff=6144, vocab=65536),
    "large": dict(width=4096, heads=32, kv=8, ssm_heads=64, mm_heads=16, ff=12288, vocab=65536),
}
RUNS = 8        # Kukulorn: four layers (attention, parallel, attention, parallel) walked twice
WINDOW = 512    # positions of the sliding window; four first tokens stay


def kukulorn_config(s):
    ff = {"kind": "dense", "ff": s["ff"]}
    att = {"heads": s["heads"], "kv_heads": s["kv"], "dim": 128, "vdim": 128, "conv": 4, "scale": 128 ** -0.5, "softcap": 50.0,
           "rot": {"base": 5e5, "dims": 64, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    left = {"heads": s["heads"], "kv_heads": s["kv"], "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "bias_max": 2048, "rel_rows": 32,
            "mask": {"size": WINDOW, "keep_first": 4}}
    right = {"heads": s["ssm_heads"], "vdim": 64, "state": 128, "groups": 1, "norm_groups": 4, "conv": 4}
    layers = [{"type": "attention", "mixer": att, "mlp": ff}, {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": ff}] * 2
    return {"architecture": "Kukulorn", "width": s["width"], "vocab": s["vocab"], "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
            "loop": {"start": 0, "stop": 4, "times": RUNS // 4}, "layers": layers}


def feruzen_config(s):
    """the same layer runs as eight Feruzen layers: where Kukulorn has attention alone, attention beside one small matrix memory
    head (that design's attention layers cannot go without; 128 values wide so that the joint output projection keeps a width the
    tuned GEMM routes take); where Kukulorn has attention beside the state-space layer, attention beside a matrix memory of the
    same state size; the same dense feed-forward on every layer"""
    ff = {"kind": "dense", "ff": s["ff"], "limit": 7.0}
    left = {"heads": s["heads"], "kv_heads": s["kv"], "dim": 128, "vdim": 128, "rot": {"base": 5e5, "dims": 64}, "scale": 128 ** -0.5}
    lone = {"left": left, "right": {"heads": 1, "dim": 16, "vdim": 128, "gate_cap": 15.0}, "left_scale": 1.0, "right_scale": 1.0}
    both = {"left": left, "right": {"heads": s["mm_heads"], "dim": 128, "vdim": 256, "gate_cap": 15.0}, "left_scale": 1.0, "right_scale": 1.0}
    four = [{"type": "parallel", "mixer": lone, "mlp": ff}, {"type": "parallel", "mixer": both, "mlp": ff}] * 2
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
    from .kukulorn import KukulornEngine
    sizes = [args.kk_size] if args.kk_size != "all" else list(SIZES)
    which = getattr(args, "kk_only", "both")
    phase = getattr(args, "kk_phase", "all")        # one phase alone gives a kernel trace of that phase only
    batches = (1, 4) if phase == "all" else (1,)
    res = {}
    for name in sizes:
        s = SIZES[name]
        res[name] = {"layer_runs": RUNS, "sizes": s}
        if which in ("both", "kukulorn"):
            res[name]["kukulorn"] = measure(KukulornEngine, kukulorn_config(s), s, args.ctx, args.ctx, batches, max(2, args.warmup), phase)
        if which in ("both", "feruzen"):
            res[name]["feruzen_equal_size"] = measure(FeruzenEngine, feruzen_config(s), s, args.ctx, args.ctx, batches, max(2, args.warmup), phase)
    print(json.dumps({"metric": "kukulorn_vs_feruzen_layer_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
                      "n_gpus": 1, "prompt_len": args.ctx, "decode_ctx": args.ctx, "results": res}))
    return 0
