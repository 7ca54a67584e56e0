"""Where the time of one decode step of the one-kernel Ladder path goes, per phase of a layer slot.

    python build.py --profile-step          # once, anywhere hipcc runs: gpt_fast/libladder_hip_prof.so
    python step_phases.py [--model gpt_ladder:ladder-70b-tp8] [--prompt 2048] [--slot 40] [--batch 1]

The profile build of the step kernel writes, per workgroup, a 100 MHz wall-clock stamp at every phase boundary of
four consecutive layer slots (lr_ladder_step_profile, profile builds only).  This script runs a few steps of the
benchmark workload (random weights, batch 1 or 2) on that library and prints, per phase, the mean / min / max duration
over the workgroups -- attention workgroups and weight-streaming workgroups separately -- the slot length, and
which workgroups (on which XCD / shader engine / CU) finish the slot last."""
import argparse
import ctypes
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

from gpt_fast import _hip  # noqa: E402

PHASES = ["slot start", "(top of loop)", "wqkv rows", "R += m, ffn norm | R += m", "w1 rows + SwiGLU | attention + merge",
          "wait for merged attention output", "wo rows", "wait for activations", "w2 rows"]
ATT_PARTS = {"attention: q wait + RoPE": (3, 10), "attention: scores": (10, 11), "attention: softmax": (11, 12),
             "attention: P.V + merge": (12, 4)}
CLOSE_PARTS = {"closing R += a, norm: words + pass 1": (8, 13), "closing: first units of the next job": (13, 15),
               "closing: sum of squares, barrier": (15, 14), "closing: pass 2": (14, 0)}


JOB_PARTS = {"wqkv": (1, 16, 17), "w1": (3, 18, 19), "wo": (5, 20, 21), "w2": (7, 22, 23)}
STALE_NAMES = ["a (closing)", "m", "merged attention output", "activations", "q/k/v", "attention partials"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", default="gpt_ladder:ladder-70b-tp8")
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--slot", type=int, default=40, help="first of the four layer slots that are stamped")
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--batch", type=int, default=1, choices=(1, 2))
    ap.add_argument("--fp8", action="store_true", help="weight-only e4m3 projections: the one-kernel step on e4m3 weights")
    ap.add_argument("--lib", default=os.path.join(HERE, "gpt_fast", "libladder_hip_prof.so"),
                    help="the profile build of the library")
    args = ap.parse_args()

    prof_lib = os.path.abspath(args.lib)
    if not os.path.exists(prof_lib):
        raise SystemExit(f"{prof_lib} is missing: python build.py --profile-step")
    _hip._LIB_PATH = prof_lib
    import benchmark as bm

    model = bm._load_model(args.model, "cuda", torch.bfloat16, seed=0, verbose=False)
    if args.fp8:
        from gpt_fast.quantize import quantize_model_fp8

        quantize_model_fp8(model)
    T = args.prompt
    B = args.batch
    model.setup_caches(B, T + 64)
    model.last_logits_only = True
    lib = _hip.load()
    set_profile = lib.lr_ladder_step_profile_fp8 if args.fp8 else lib.lr_ladder_step_profile
    set_profile.restype = ctypes.c_size_t
    set_profile.argtypes = [ctypes.c_void_p, ctypes.c_int]
    with torch.no_grad():
        prompt = torch.randint(0, model.config.vocab_size, (T,), device="cuda")
        first = bm.prefill(model, prompt.view(1, -1).repeat(B, 1), torch.arange(T, device="cuda", dtype=torch.int32),
                           greedy=True).clone()
        pos = torch.tensor([T], dtype=torch.int32, device="cuda")
        for _ in range(3):
            model(first.view(B, 1), pos)
        nbytes = set_profile(None, 0)
        buf = torch.zeros(nbytes // 8, dtype=torch.int64, device="cuda")
        set_profile(buf.data_ptr(), args.slot)
        # two single stamped steps first: are the same workgroups slow in the same slot of different steps?
        snaps = []
        for _ in range(2):
            model(first.view(B, 1), pos)
            torch.cuda.synchronize()
            snaps.append(buf.cpu().numpy().reshape(-1, 4, 32).astype(np.float64) * 0.01)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            model(first.view(B, 1), pos)
        e1.record()
        torch.cuda.synchronize()
        set_profile(None, 0)
    model.check_device_errors()
    print(f"{args.model}{' (e4m3 weights)' if args.fp8 else ''}, batch {B}, position {T}: {e0.elapsed_time(e1) / args.steps:.3f} ms per step (profile build, eager launches)")
    NP = 32   # stamps per workgroup and slot (PROF_POINTS of the kernel)
    a = buf.cpu().numpy().reshape(-1, 4, NP).astype(np.float64) * 0.01   # [workgroup][slot][stamp] in microseconds
    nwg = a.shape[0]
    s = 1   # second of the four stamped slots
    na = int((a[:, s, 10] > 0).sum())   # only attention workgroups write the attention stamps (the first `na`)
    groups = {"weight-streaming workgroups": slice(na, nwg), "attention workgroups": slice(0, na)}
    print(f"layer slots {args.slot}..{args.slot + 3}; {nwg} workgroups, {na} of them attention workgroups; durations in microseconds, "
          "per workgroup averaged over the four slots")
    for gname, sl in groups.items():
        print(f"  {gname}")
        for k in range(2, len(PHASES)):
            d = (a[sl, :, k] - a[sl, :, k - 1]).mean(axis=1)
            print(f"    {PHASES[k]:42s} mean {d.mean():6.2f}  min {d.min():6.2f}  max {d.max():6.2f}")
        for nm, (k0, k1) in CLOSE_PARTS.items():
            d = (a[sl, :, k1] - a[sl, :, k0]).mean(axis=1)
            print(f"    {nm:42s} mean {d.mean():6.2f}  min {d.min():6.2f}  max {d.max():6.2f}")
    print("  inside the projections (weight-streaming workgroups): unit loop | reduction + epilogue")
    for nm, (k0, k1, k2) in JOB_PARTS.items():
        d0, d1 = (a[na:, :, k1] - a[na:, :, k0]).mean(axis=1), (a[na:, :, k2] - a[na:, :, k1]).mean(axis=1)
        print(f"    {nm:42s} mean {d0.mean():6.2f} | {d1.mean():5.2f}   max {d0.max():6.2f} | {d1.max():5.2f}")
    for nm, k0, k1 in (("wqkv: entry -> first unit wanted", 1, 30), ("wo: entry -> first unit wanted", 5, 31)):
        d = (a[na:, :, k1] - a[na:, :, k0]).mean(axis=1)
        print(f"    {nm:42s} mean {d.mean():6.2f}   max {d.max():6.2f}")
    cnt = buf.cpu().numpy().reshape(-1, 4, NP)[:, :, 24:30].sum(axis=(0, 1)) / (4.0 * args.steps)
    print("  exchanged words not there at the first look, per slot, summed over the workgroups: "
          + ", ".join(f"{n} {c:.1f}" for n, c in zip(STALE_NAMES, cnt)))
    for nm, (k0, k1) in ATT_PARTS.items():
        d = (a[:na, :, k1] - a[:na, :, k0]).mean(axis=1)
        print(f"    {nm:42s} mean {d.mean():6.2f}  min {d.min():6.2f}  max {d.max():6.2f}")
    lens = [(a[:, j + 1, 1] - a[:, j, 1]).mean() for j in range(3)]
    print("  slot length (loop top to loop top), three consecutive slots: " + ", ".join(f"{x:.2f}" for x in lens))
    ends = a[:, s, 8] - a[:, s, 1].min()
    print(f"  w2 finish time after the first workgroup entered the slot: mean {ends.mean():.2f}, last {ends.max():.2f}")
    # stamp 9 holds where the workgroup runs: XCC_ID above the low 16 bits of HW_ID (CU [11:8], SH [12], SE [15:13])
    hw = buf.cpu().numpy().reshape(-1, 4, NP)[:, s, 9]
    xcc, se, cu = (hw >> 16) & 0xF, (hw >> 13) & 0x7, (hw >> 8) & 0xF
    last = np.argsort(ends)[-6:][::-1]
    print("  the six workgroups that finish w2 last (workgroup: XCD / shader engine / CU, lag behind the mean):")
    print("    " + ", ".join(f"{w}: {xcc[w]}/{se[w]}/{cu[w]} +{ends[w] - ends.mean():.1f}" for w in last))
    lag1 = a[last, s, 4] - a[:, s, 4].mean()
    print("    the same six at the end of w1 | attention: " + ", ".join(f"+{x:.1f}" for x in lag1))
    d0 = snaps[0][na:, :, 4] - snaps[0][na:, :, 3]
    d1 = snaps[1][na:, :, 4] - snaps[1][na:, :, 3]
    cc = [float(np.corrcoef(d0[:, j], d1[:, j])[0, 1]) for j in range(4)]
    cx = float(np.corrcoef(d0[:, 0], d0[:, 1])[0, 1])
    print("  w1 duration per workgroup, correlation between two steps in the same slot (four slots): "
          + ", ".join(f"{c:.2f}" for c in cc) + f"; between neighbouring slots of one step: {cx:.2f}")
    print("  mean w2 finish per XCD: " + ", ".join(f"{ends[xcc == x].mean():.1f}" for x in range(int(xcc.max()) + 1)))


if __name__ == "__main__":
    main()
