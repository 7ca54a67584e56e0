"""Where the time of one launch of the weight-streaming band kernel (lr_linear_multi, decode batches) goes.

    python build.py --profile-bands         # once, anywhere hipcc runs: gpt_fast/libladder_hip_bandprof.so
    python band_phases.py [--rows 8]

The profile build of the band kernel writes, per wave, a 100 MHz wall-clock stamp at six points: entry, first
requests made, first chunk of weights in LDS, end of the K loop, partial sums exchanged, end.  This script launches
the projections of one decoder layer at the shapes of the benchmark workloads -- each on weights that no earlier
launch has touched, so that they come from HBM as they do inside a step -- and prints, per launch, how long the
workgroups take between the stamps, when they enter and when they end, relative to the first entry of the launch."""
import argparse
import ctypes
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

from gpt_fast import _hip  # noqa: E402

NAMES = ["entry -> first requests made", "-> first chunk in LDS", "-> end of the K loop", "-> partial sums exchanged",
         "-> end (sum, epilogue, store)"]
MAX_WG = 4096


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--rows", type=int, default=8, help="input rows (sequences of the decode batch) of the 70B launches")
    ap.add_argument("--lib", default=os.path.join(HERE, "gpt_fast", "libladder_hip_bandprof.so"),
                    help="the profile build of the library")
    args = ap.parse_args()
    prof_lib = os.path.abspath(args.lib)
    if not os.path.exists(prof_lib):
        raise SystemExit(f"{prof_lib} is missing: python build.py --profile-bands")
    _hip._LIB_PATH = prof_lib
    lib = _hip.load()
    lib.lr_band_profile.restype = ctypes.c_longlong
    lib.lr_band_profile.argtypes = [ctypes.c_void_p, ctypes.c_int]
    dev = "cuda"
    nbytes = lib.lr_band_profile(None, MAX_WG)
    assert nbytes > 0, nbytes
    prof = torch.zeros(nbytes // 8, dtype=torch.int64, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(0)

    def rnd(*s):
        return (torch.randn(*s, device=dev, generator=g) * 0.02).to(torch.bfloat16)

    def out(m, n):
        return torch.empty(m, n, dtype=torch.bfloat16, device=dev)

    def qkv(M, D, Hq, Hkv, hd, S, T):
        table = rnd(2 * T, hd // 2, 2)
        pos = torch.tensor([T], dtype=torch.int32, device=dev)
        kc = torch.zeros(M, Hkv, S, hd, dtype=torch.bfloat16, device=dev)
        vc = torch.zeros_like(kc)
        n = (Hq + 2 * Hkv) * hd
        return lambda: ((rnd(M, D), rnd(n, D), out(M, n), _hip.rope_kv_epilogue(table, pos, kc, vc, Hq, Hkv, hd)),)

    def wo_w2(M, D, Q, I):
        return lambda: ((rnd(M, Q), rnd(D, Q), out(M, D), _hip.EPI_NONE), (rnd(M, I), rnd(D, I), out(M, D), _hip.EPI_NONE))

    def up_gate(M, D, I):
        return lambda: ((rnd(M, D), rnd(2 * I, D), out(M, I), _hip.EPI_SWIGLU),)

    def run(tag, make, reps=6):
        sets = [make() for _ in range(reps)]   # fresh weights per launch: nothing of them is in L2
        for st in sets[:-1]:
            _hip.linear_multi(*st)
        torch.cuda.synchronize()
        prof.zero_()
        torch.cuda.synchronize()
        assert lib.lr_band_profile(prof.data_ptr(), MAX_WG) > 0
        _hip.linear_multi(*sets[-1])
        torch.cuda.synchronize()
        lib.lr_band_profile(None, 0)
        t = prof.view(-1, 4, 8).cpu().double() * 0.01   # [workgroup][wave][stamp], microseconds
        nwg = int((t[:, 0, 0] != 0).sum().item())
        t = t[:nwg]
        t0 = t[:, :, 0].min()
        w0 = t[:, 0, :]                                 # wave 0 of every workgroup
        print(f"--- {tag}: {nwg} workgroups; first entry to last end {(t[:, :, 5].max() - t0):.2f} us")
        print(f"    entry after the first entry       mean {(w0[:, 0] - t0).mean():6.2f}               max {(w0[:, 0] - t0).max():6.2f}")
        for k, n in enumerate(NAMES):
            d = w0[:, k + 1] - w0[:, k]
            print(f"    {n:33s} mean {d.mean():6.2f}  min {d.min():6.2f}  max {d.max():6.2f}")
        le = t[:, :, 3]
        print(f"    end of the K loop, last wave of a workgroup after its first: mean {(le.max(1).values - le.min(1).values).mean():.2f}")
        e = w0[:, 5] - t0
        print(f"    end after the first entry         mean {e.mean():6.2f}  min {e.min():6.2f}  max {e.max():6.2f}")

    M = args.rows
    run(f"70B TP8 shard, q/k/v (1280 x 8192, RoPE + cache epilogue), {M} rows", qkv(M, 8192, 8, 1, 128, 2304, 2048))
    run(f"70B TP8 shard, up/gate (7168 x 8192, SwiGLU epilogue), {M} rows", up_gate(M, 8192, 3584))
    run(f"70B TP8 shard, wo (8192 x 1024) next to w2 (8192 x 3584), {M} rows", wo_w2(M, 8192, 1024, 3584))
    run("70B TP8 shard, wo next to w2, 64 rows", wo_w2(64, 8192, 1024, 3584))
    run("Ladder-8B, q/k/v (6144 x 4096), 16 rows", qkv(16, 4096, 32, 8, 128, 1280, 1024))
    run("Ladder-8B, wo (4096 x 4096) next to w2 (4096 x 14336), 16 rows", wo_w2(16, 4096, 4096, 14336))


if __name__ == "__main__":
    main()
