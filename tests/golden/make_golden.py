"""Writes tests/golden/tiny_*.npz: inputs and expected outputs of the oracle on a tiny configuration.

    python tests/golden/make_golden.py

The reference ships no golden vectors for this path and cannot be imported here (it needs CUDA,
NCCL, flash_attn and liger_kernel at import time), so these vectors are written by the oracle
(oracle/ladder_oracle.py, PyTorch CPU, bf16 storage).  They freeze the oracle's behaviour -- a later
edit that changes a rounding point or a schedule shows up as a fixture mismatch on the CPU -- and
give the GPU tests a committed target that does not depend on running the oracle on the GPU box.

Each file holds, for one model family: the configuration, every parameter as raw bf16 bits
(uint16), the prompt, and for B = 2 identical rows the greedy tokens and the bf16 logits of the
last prompt position and of every decode step."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import ladder_oracle as O  # noqa: E402

CFG = dict(block_size=64, vocab_size=256, n_layer=3, n_head=2, n_local_heads=1, dim=128, intermediate_size=256,
           rope_base=10000)
B, T, NEW = 2, 12, 6


def bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).contiguous().view(torch.int16).numpy().view(np.uint16)


def main():
    torch.set_num_threads(1)
    for family in ("ladder", "dense", "desync", "parallel"):
        kw = dict(CFG)
        if family == "desync":
            kw["reduce_pattern"] = [{"attention": False, "mlp": True}, {"attention": True, "mlp": False},
                                    {"attention": False, "mlp": False}]
        cfg = O.OracleConfig(**kw)
        P = O.init_params(cfg, family, seed=7, dtype=torch.bfloat16, std=0.25)  # large enough for the blocks to matter
        g = torch.Generator()
        g.manual_seed(11)
        prompt = torch.randint(0, cfg.vocab_size, (T,), generator=g)
        tokens, logits = O.generate(cfg, P, prompt, NEW, B, family)
        out = {"param:" + k: bits(v) for k, v in P.items()}
        out["prompt"] = prompt.numpy().astype(np.int64)
        out["tokens"] = tokens.numpy().astype(np.int32)                       # [B, NEW]
        out["logits"] = np.stack([bits(l) for l in logits])                   # [NEW, B, V] bf16 bits
        out["shape"] = np.array([B, T, NEW], dtype=np.int64)
        path = os.path.join(HERE, f"tiny_{family}.npz")
        np.savez_compressed(path, **out)
        print(path, os.path.getsize(path) // 1024, "KiB", "tokens", tokens[0].tolist())


if __name__ == "__main__":
    main()
