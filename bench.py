"""Headline benchmark: batch-1 greedy decode of one TP=8 rank shard of Ladder-70B on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--no-cpu-baseline]

A "step" is one decode step (one new token per sequence) of the whole per-rank forward pass,
replayed as a captured hipGraph: embedding -> 80 ladder blocks -> final add/norm -> vocab-shard
lm_head -> argmax -> device-side token/position hand-over.  Weights are random N(0, 0.02) bf16
(seed 0), the prompt is 2048 uniform-random ids; the prompt is prefilled before the timed region
so the KV cache has its real length, and the timed steps start at position 2048.  Everything the
steps read is resident in HBM when the clock starts.

Prints ONE JSON line.  `value` = decoded tokens per second (whole job = the one GPU).
`roofline`   : the dominant kernel.  For the ladder model at batch <= 2 that is k_ladder_step, ONE
               persistent launch per decode step; `achieved` = algorithmic bytes per launch (all
               weights and gains once + valid KV + KV write + embedding rows + logits) / its mean
               launch duration, measured here with HIP events around back-to-back launches on the
               launch stream.  `traffic` = HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE
               counter runs (a constant recorded from those runs, or null).  Other models / batches
               run the per-op path, whose dominant kernel is the up/gate projection (timed alone here:
               the GEMV up to batch 4, the matrix-core band kernel above).
               `measured_read_ceiling` = GB/s of a plain streaming read of 8 GiB by every CU
               (lr_stream_read) on this machine in the same run; `frac` is against the nominal
               8 TB/s, `frac_of_measured_ceiling` against that.
`step_roofline`: the same ratio for the whole decode step as replayed from the hipGraph (kernel +
               token hand-over): algorithmic bytes per step / measured step time.
`cpu_baseline`: the oracle (a PyTorch-CPU restatement of the reference; the reference itself cannot
               run without CUDA + NCCL) timed on this machine's host cores on the reference's
               CPU-sized case: Ladder-1B fp32, batch 1, 128-token prompt, greedy decode.  `cores` =
               threads used (the process's CPU share: OMP_NUM_THREADS when set, else every core),
               `host_cpus` = os.cpu_count().
Measured in the same run and reported as extra keys (not the headline; --no-extras skips them):
`batched`     : the same rank shard at batch 2 (one-kernel step), 4, 8 and 64, the 8B model at batch 1 (one-kernel
               step) and 16 (prompt 1024) and the 405B rank shard at batch 16 (context 4096) -- per-op kernels unless noted,
               hipGraph replay: ms per step, tok/s, algorithmic GB/s and its fraction of 8 TB/s; `traffic` = HBM
               bytes per step from counter runs where one was made.
`fp8`         : the same shard with weight-only e4m3 projections at batch 1 (the one-kernel step on e4m3 weights)
               and batch 8 (per-op kernels): ms per step and the fraction of 8 TB/s on ITS algorithmic bytes
               (one byte per weight + scales).
`prefill`     : Ladder-8B, batch 32 x 2048 prompt tokens, causal prefill with last-position logits:
               seconds, algorithmic TFLOP/s and the fraction of 2.5 PFLOP/s (dense bf16 MFMA peak)."""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ladder-residual-inference_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0   # dense bf16
# HBM bytes one launch of the dominant kernel moves, per workload (model, batch, prompt), from the rocprofv3
# FETCH_SIZE / WRITE_SIZE counter runs summarised under profiles/; workloads without a counter run report null.
TRAFFIC_BYTES_PER_LAUNCH = {
    ("gpt_ladder:ladder-70b-tp8", 1, 2048): 17.585e9,    # k_ladder_step, 1.007 x algorithmic
    # the up/gate projection alone (the kernel the batched workloads' roofline object is measured on):
    ("gpt_ladder:ladder-70b-tp8", 8, 2048): 118.75e6,    # k_stream_gemm<16,2>, 256 bands: 1.009 x algorithmic
    ("gpt_ladder:ladder-70b-tp8", 64, 2048): 126.46e6,   # k_stream_gemm<64,2>, the decode step's 224 bands: 1.06 x
}
# HBM bytes of a whole decode step through the per-op kernels (all its launches), from the same kind of counter runs
STEP_TRAFFIC_BYTES = {
    ("gpt_ladder:ladder-70b-tp8", 8, 2048): 22.41e9,     # 1.24 x algorithmic
    ("gpt_ladder:ladder-70b-tp8", 64, 2048): 30.46e9,    # 1.34 x algorithmic
}


def cpu_baseline(new_tokens=32, repeats=2):
    """Oracle on the host cores, config 1 of the benchmark set.  Returns the cpu_baseline object."""
    import torch

    from oracle import ladder_oracle as O

    host_cpus = os.cpu_count() or 1
    # the process may own only a share of the host (the harness exports it as OMP_NUM_THREADS): more threads than
    # that only fight each other
    cores = min(host_cpus, int(os.environ.get("OMP_NUM_THREADS", host_cpus)))
    torch.set_num_threads(cores)
    cfg = O.OracleConfig(block_size=2048, vocab_size=128256, n_layer=16, n_head=32, n_local_heads=8, dim=2048,
                         intermediate_size=8192, rope_base=500000)
    dev = "cuda" if torch.cuda.is_available() else "cpu"   # generate the random weights fast, compute on the CPU
    P = {k: v.float().cpu() for k, v in O.init_params(cfg, seed=0, dtype=torch.float32, device=dev).items()}
    g = torch.Generator()
    g.manual_seed(1)
    prompt = torch.randint(0, cfg.vocab_size, (128,), generator=g)
    O.generate(cfg, P, prompt, 2, 1)  # warm the allocator and thread pool
    dec, pre = [], []
    for _ in range(repeats):
        tm = {}
        O.generate(cfg, P, prompt, new_tokens, 1, timers=tm)
        dec.append(tm["decode_latency"] / (new_tokens - 1))
        pre.append(tm["prefill_latency"])
    ms = 1e3 * sum(dec) / len(dec)
    return {"value": round(1e3 / ms, 3), "unit": "tok/s", "cores": cores, "host_cpus": host_cpus, "kind": "port",
            "ms_per_token": round(ms, 3), "prefill_s": round(sum(pre) / len(pre), 3),
            "sample": f"oracle (PyTorch CPU fp32) on Ladder-1B (dim 2048, 16 layers, 32q/8kv, FFN 8192, vocab 128256), "
                      f"B=1, prompt 128, greedy decode of {new_tokens} tokens, {repeats} runs"}


def decode_run(bm, model, prompt, B, T, K, W):
    """Prefill the prompt at batch B, capture the decode step, run W untimed + K timed steps from position T.
    Returns (ms per step, first token tensor, DecodeGraph)."""
    import torch

    new = max(K, W) + 1
    model.max_seq_length = -1            # new caches for this batch size
    model.setup_caches(B, T + max(new, 128))
    rows = prompt.view(1, -1).repeat(B, 1)
    first = bm.prefill(model, rows, torch.arange(T, device=prompt.device, dtype=torch.int32), greedy=True).clone()
    dg = bm.get_cuda_graphs_for_decode(model, prompt, B, new, first, greedy=True)
    dg.reset(first)
    for _ in range(W):
        dg.replay()
    dg.reset(first)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        dg.replay()
    torch.cuda.synchronize()
    ms = 1e3 * (time.perf_counter() - t0) / K
    model.check_device_errors()
    return ms, first, dg


def extra_batched(bm, model, prompt, T, batches=(2, 4, 8, 64), K=32, W=5):
    """The headline shard at other batch sizes (2: the one-kernel step; from 3 on the per-op kernels; 4, 8 and 64 are
    those of the benchmark set)."""
    cfg = model.config
    out = []
    for B in batches:
        ms, _, dg = decode_run(bm, model, prompt, B, T, K, W)
        nbytes = sum(bm.decode_bytes_per_step(cfg, B, T + i) for i in range(K)) / K
        gbps = nbytes / (ms * 1e-3) / 1e9
        out.append({"model": "gpt_ladder:ladder-70b-tp8", "batch": B, "prompt_len": T, "ms_per_step": round(ms, 4),
                    "tok_per_s": round(B * 1e3 / ms, 1), "bytes_per_step": int(nbytes), "achieved_GBps": round(gbps, 1),
                    "frac": round(gbps / HBM_PEAK_GBPS, 4), "steps": K,
                    "traffic": STEP_TRAFFIC_BYTES.get(("gpt_ladder:ladder-70b-tp8", B, T))})
        del dg
    return out


def extra_model_decode(bm, name, B, T, K=16, W=3):
    """Another decode configuration of the benchmark set, on a model of its own (random weights)."""
    import torch

    model = bm._load_model(name, "cuda", torch.bfloat16, seed=0, verbose=False)
    model.last_logits_only = True
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    prompt = torch.randint(0, model.config.vocab_size, (T,), device="cuda", generator=g)
    ms, _, dg = decode_run(bm, model, prompt, B, T, K, W)
    nbytes = sum(bm.decode_bytes_per_step(model.config, B, T + i) for i in range(K)) / K
    gbps = nbytes / (ms * 1e-3) / 1e9
    del dg, model
    torch.cuda.empty_cache()
    return {"model": name, "batch": B, "prompt_len": T, "ms_per_step": round(ms, 4), "tok_per_s": round(B * 1e3 / ms, 1),
            "bytes_per_step": int(nbytes), "achieved_GBps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4),
            "steps": K}


def fp8_bytes_per_step(cfg, B, pos):
    """decode_bytes_per_step with one byte per projection weight plus a bf16 scale per output row."""
    D, L, hd = cfg.dim, cfg.n_layer, cfg.head_dim
    Hq, Hkv, I, V = cfg.n_head_local, cfg.n_kv_local, cfg.ffn_local, cfg.output_rows
    nqkv = (Hq + 2 * Hkv) * hd
    w = L * (D * nqkv + D * Hq * hd + D * 2 * I + I * D) + V * D                   # one byte each
    scales = 2 * (L * (nqkv + D + 2 * I + D) + V)
    gains = 2 * (L * 2 * D + D)
    kv = 2 * (L * B * 2 * Hkv * hd * (pos + 1) + L * B * 2 * Hkv * hd) + 2 * B * D
    return w + scales + gains + kv


def extra_fp8(bm, model, prompt, T, K=32, W=5):
    """Weight-only e4m3 projections on the headline shard, batch 1 and 8.  Quantises `model` in place (call it last)."""
    from gpt_fast.quantize import quantize_model_fp8

    quantize_model_fp8(model)
    res = []
    for B, kernels in ((1, "one-kernel step (lr_ladder_decode_step_fp8), hipGraph replay"),
                       (8, "per-op (fp8 matrix-core bands), hipGraph replay")):
        ms, _, dg = decode_run(bm, model, prompt, B, T, K, W)
        if B == 1 and model._fused_step(B) is None:
            kernels = "per-op (fp8 matrix-vector kernel), hipGraph replay"
        nbytes = sum(fp8_bytes_per_step(model.config, B, T + i) for i in range(K)) / K
        gbps = nbytes / (ms * 1e-3) / 1e9
        res.append({"batch": B, "ms_per_step": round(ms, 4), "tok_per_s": round(B * 1e3 / ms, 1),
                    "bytes_per_step": int(nbytes), "achieved_GBps": round(gbps, 1),
                    "frac": round(gbps / HBM_PEAK_GBPS, 4), "steps": K, "kernels": kernels})
        del dg
    out = res[0]
    out["batch8"] = res[1]
    return out


def extra_prefill(bm, B=32, T=2048, reps=2):
    """Config 4: Ladder-8B, B x T prompt tokens, causal prefill, logits of the last position."""
    import torch

    model = bm._load_model("gpt_ladder:ladder-8b", "cuda", torch.bfloat16, seed=0, verbose=False)
    model.last_logits_only = True
    c = model.config
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    rows = torch.randint(0, c.vocab_size, (T,), device="cuda", generator=g).view(1, -1).repeat(B, 1)
    pos = torch.arange(T, device="cuda", dtype=torch.int32)
    model.setup_caches(B, T + 8)
    bm.prefill(model, rows, pos, greedy=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        bm.prefill(model, rows, pos, greedy=True)
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / reps
    model.check_device_errors()
    D, L, hd, Hq, Hkv, I, V = c.dim, c.n_layer, c.head_dim, c.n_head_local, c.n_kv_local, c.ffn_local, c.output_rows
    lin = 2 * B * T * L * (D * (Hq + 2 * Hkv) * hd + D * Hq * hd + 3 * D * I) + 2 * B * V * D
    att = L * B * Hq * 2 * hd * T * T
    tf = (lin + att) / sec / 1e12
    return {"workload": f"gpt_ladder:ladder-8b, batch {B} x {T} prompt tokens, causal prefill, last-position logits",
            "seconds": round(sec, 4), "flop": int(lin + att), "achieved_TFLOPs": round(tf, 1),
            "peak_TFLOPs": MFMA_PEAK_TFLOPS, "frac": round(tf / MFMA_PEAK_TFLOPS, 4),
            "prompt_tok_per_s": round(B * T / sec, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=127)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--model", type=str, default="gpt_ladder:ladder-70b-tp8")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the extra keys (other batch sizes, fp8 weights, the prefill-heavy configuration)")
    ap.add_argument("--per-op", action="store_true",
                    help="decode with one kernel per operation (captured in the hipGraph) instead of the persistent "
                         "one-kernel step: the comparison point, not the headline")
    ap.add_argument("--fp8", action="store_true",
                    help="weight-only e4m3 projections (gpt_fast.quantize): a profiling aid, not the headline")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (reads 1 GiB, writes 1 GiB) a few times: under "
                         "rocprofv3 --pmc its FETCH_SIZE / WRITE_SIZE readings calibrate the counters' unit")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures ONE tensor-parallel rank's shard on ONE GPU (partial sums stay local, no "
              "collectives); --gpus must be 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    import benchmark as bm
    from gpt_fast import _hip

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    _hip.load()
    dev = "cuda"
    B, T, K, W = args.batch, args.prompt, args.steps, args.warmup
    model = bm._load_model(args.model, dev, torch.bfloat16, seed=0, verbose=False)
    model.last_logits_only = True          # prefill is set-up here, not the timed region
    if args.per_op:
        model.use_fused_step = False
    if args.fp8:
        from gpt_fast.quantize import quantize_model_fp8

        quantize_model_fp8(model)
    cfg = model.config
    new = max(K, W, 127) + 1
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    prompt = torch.randint(0, cfg.vocab_size, (T,), device=dev, generator=g)
    model.setup_caches(B, T + new)

    # ---- set-up: prefill the prompt (eager), capture the decode step
    rows = prompt.view(1, -1).repeat(B, 1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    first = bm.prefill(model, rows, torch.arange(T, device=dev, dtype=torch.int32), greedy=True).clone()
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    dg = bm.get_cuda_graphs_for_decode(model, prompt, B, new, first, greedy=True)

    if args.calibrate_copy:
        src = torch.zeros(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- W untimed steps, then exactly K timed steps from position T
    dg.reset(first)
    for _ in range(W):
        dg.replay()
    dg.reset(first)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        dg.replay()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    model.check_device_errors()   # raises if any timed step did not do its work (expired wait, position out of range)
    ms_per_step = 1e3 * elapsed / K
    tokens = dg.history[0, : min(K, 16)].tolist()

    bytes_per_step = fp8_bytes_per_step if args.fp8 else bm.decode_bytes_per_step
    step_bytes = sum(bytes_per_step(cfg, B, T + i) for i in range(K)) / K
    step_gbps = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- dominant kernel, timed with HIP events on the stream it is launched on (torch's current stream)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fused = getattr(model, "use_fused_step", False) and hasattr(model, "decode_step_fused") and \
        model._fused_step(B) is not None
    if fused:
        # the whole step is ONE kernel (k_ladder_step): algorithmic bytes per launch = bytes per step
        pos = torch.tensor([T], dtype=torch.int32, device=dev)
        tok = first.view(B, 1).to(torch.int32).contiguous()
        for _ in range(3):
            model.decode_step_fused(tok, pos)
        reps = 30
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(reps):
            model.decode_step_fused(tok, pos)
        ev1.record()
        torch.cuda.synchronize()
        k_us = 1e3 * ev0.elapsed_time(ev1) / reps
        model.check_device_errors()
        k_bytes = bytes_per_step(cfg, B, T)
        k_name = (f"k_ladder_step (one persistent launch = the whole decode step at position {T}: "
                  f"{cfg.n_layer} layers + lm_head, M={B}{', e4m3 weights' if args.fp8 else ''})")
    else:
        # per-op path: the weight-streaming GEMV on the w1 (up+gate) projection, a distinct matrix per launch
        w1s = [blk.feed_forward.w1.weight for blk in model.layers] if hasattr(model.layers[0], "feed_forward") else \
            [blk.attention.wqkv1.weight for blk in model.layers]
        N, Kdim = w1s[0].shape
        x = torch.randn(B, Kdim, device=dev).to(torch.bfloat16)
        y = torch.empty(B, N, device=dev, dtype=torch.bfloat16)
        if args.fp8:
            scs = [(blk.feed_forward.w1 if hasattr(blk, "feed_forward") else blk.attention.wqkv1).scales
                   for blk in model.layers]
            run = lambda i: _hip.linear_fp8_multi((x, w1s[i], scs[i], y, _hip.EPI_NONE)) if B <= 16 else \
                _hip.linear_fp8(x, w1s[i], scs[i], y)
        else:
            run = lambda i: _hip.linear(x, w1s[i], y)
        for i in range(8):
            run(i)
        reps = 3
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(reps):
            for i in range(len(w1s)):
                run(i)
        ev1.record()
        torch.cuda.synchronize()
        k_us = 1e3 * ev0.elapsed_time(ev1) / (reps * len(w1s))
        wbytes = 1 if args.fp8 else 2
        k_bytes = wbytes * N * Kdim + 2 * (B * Kdim + B * N)
        kern = ("k_gemv_fp8_multi" if B == 1 else "k_stream_gemm (e4m3 bands)") if args.fp8 else \
            ("k_gemv" if B <= 4 else "k_stream_gemm")
        k_name = f"{kern} (w1 up+gate projection, [{N} x {Kdim}] {'e4m3' if args.fp8 else 'bf16'}, M={B})"
    k_gbps = k_bytes / (k_us * 1e-6) / 1e9

    # ---- the read rate this machine reaches: a plain streaming read of 8 GiB by every CU
    ceil_buf = torch.empty(8 << 30, dtype=torch.uint8, device=dev)
    ceil_buf.view(torch.int32).fill_(0x01010101)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    for _ in range(2):
        _hip.stream_read(ceil_buf, sink)
    torch.cuda.synchronize()
    ev0.record()
    for _ in range(5):
        _hip.stream_read(ceil_buf, sink)
    ev1.record()
    torch.cuda.synchronize()
    ceiling_gbps = 5 * ceil_buf.numel() / (ev0.elapsed_time(ev1) * 1e-3) / 1e9
    del ceil_buf

    out = {
        "metric": "decode_tokens_per_sec", "value": round(B * 1e3 / ms_per_step, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16 (e4m3 weights)" if args.fp8 else "bf16",
        "data": "synthetic",
        "config": {"workload": f"{args.model} rank shard (dim {cfg.dim}, {cfg.n_layer} layers, {cfg.n_head_local} q / "
                               f"{cfg.n_kv_local} kv heads, FFN {cfg.ffn_local}, lm_head rows {cfg.output_rows}), "
                               f"batch {B}, prompt {T}, greedy decode, hipGraph replay per step"
                               + (", one kernel per operation" if args.per_op else "")
                               + (", weight-only e4m3 projections" if args.fp8 else ""),
                   "batch": B, "prompt_len": T, "virtual_tp": cfg.tp_world_size},
        "ms_per_token": round(ms_per_step, 4),
        "prefill_s": round(prefill_s, 4),
        "roofline": {"bound": "hbm", "kernel": k_name,
                     "achieved": round(k_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(k_gbps / HBM_PEAK_GBPS, 4),
                     "traffic": TRAFFIC_BYTES_PER_LAUNCH.get((args.model, B, T)) if (fused or B > 4) and not args.fp8 else None,
                     "bytes_per_launch": int(k_bytes), "avg_launch_us": round(k_us, 3),
                     "measured_read_ceiling": round(ceiling_gbps, 1),
                     "frac_of_measured_ceiling": round(k_gbps / ceiling_gbps, 4)},
        "step_roofline": {"bound": "hbm", "achieved": round(step_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                          "frac": round(step_gbps / HBM_PEAK_GBPS, 4), "bytes_per_step": int(step_bytes)},
        "first_tokens": tokens,
    }
    del dg
    if not args.no_extras and args.model == "gpt_ladder:ladder-70b-tp8" and B == 1:
        out["batched"] = extra_batched(bm, model, prompt, T)
        out["fp8"] = extra_fp8(bm, model, prompt, T)
        del model
        torch.cuda.empty_cache()
        out["prefill"] = extra_prefill(bm)
        # the other decode configurations of the benchmark set: the 8B model at batch 16, the 405B rank shard at batch 16
        out["batched"].append(extra_model_decode(bm, "gpt_ladder:ladder-8b", 1, 1024, K=32, W=5))   # one-kernel step
        out["batched"].append(extra_model_decode(bm, "gpt_ladder:ladder-8b", 16, 1024))
        out["batched"].append(extra_model_decode(bm, "gpt_ladder:ladder-405b-tp8", 16, 4096))
    else:
        del model
    torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
