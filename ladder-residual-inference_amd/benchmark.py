"""Throughput benchmark for one tensor-parallel rank's shard of a Ladder / dense / desync / parallel
transformer on one MI355X -- the command line of the reference's benchmark.py on the HIP backend.

Kept from the reference (benchmark.py:495-540): --model_name family:config, --prompt_length,
--num_samples, --max_new_tokens, --batch_size, --top_k, --temperature, --compile,
--compile_prefill, --cuda_graph, --use_flash_attention, --profile, --device; five untimed warm-up
generations; prefill and decode timed separately between device synchronisations; the printed
metric lines.  Added: --greedy (argmax on the device, lowest index on ties), --seed (weights
N(0, 0.02) for every parameter and the prompt come from one seeded device generator),
--virtual_tp / --tp_rank / --shard_vocab (build the layers at 1/N size without any process group),
--last_logits_only, --json.

There is no compiler in this build: --compile and --cuda_graph both select hipGraph replay of a
captured decode step (the captured step also copies the new token and advances the position on
the device, so the replay loop issues nothing but graph launches); without either flag the
kernels are launched eagerly through the C ABI."""
import argparse
import contextlib
import json
import sys
import time
from pathlib import Path
from typing import Optional, Tuple

import torch

sys.path.insert(0, str(Path(__file__).parent.resolve()))

from gpt_fast import GPTDense, GPTDesync, GPTLadder, GPTParallel, _hip, set_virtual_tp  # noqa: E402
from gpt_fast.utils import _get_model_size, set_flash_attention  # noqa: E402

default_device = "cuda" if torch.cuda.is_available() else "cpu"

_MODELS = {
    "gpt_dense": GPTDense,
    "gpt_desync": GPTDesync,
    "gpt_parallel": GPTParallel,
    "gpt_ladder": GPTLadder,
}

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, vendor figure


def print_rank_0(*args, **kwargs):
    print(*args, **kwargs, flush=True)


def device_sync(device):
    if "cuda" in str(device):
        torch.cuda.synchronize(device)


# ------------------------------------------------------------------------------------------------
# sampling
# ------------------------------------------------------------------------------------------------

def multinomial_sample_one_no_sync(probs_sort):
    """Exponential-race sampling without a host synchronisation: argmax(p / Exp(1))."""
    noise = torch.empty_like(probs_sort).exponential_(1)
    return torch.argmax(probs_sort / noise, dim=-1, keepdim=True).to(dtype=torch.int)


def logits_to_probs(logits, temperature: float = 1.0, top_k: Optional[int] = None):
    logits = logits / max(temperature, 1e-5)
    if top_k is not None:
        kth = torch.topk(logits, min(top_k, logits.size(-1)))[0][..., -1:]
        logits = torch.where(logits < kth, -float("Inf"), logits)
    return torch.nn.functional.softmax(logits, dim=-1)


def sample(logits, temperature: float = 1.0, top_k: Optional[int] = None, greedy: bool = False, model=None):
    """Next token from the logits of the last position -> (int32 [B, 1], probabilities or None)."""
    if greedy:
        if model is not None:
            return model.greedy_next(logits), None            # lr_argmax on the device
        return torch.argmax(logits[:, -1], dim=-1, keepdim=True).to(torch.int), None
    if model is not None and logits.is_cuda and logits.dtype == torch.bfloat16:
        return model.sample_next(logits, temperature, top_k)  # lr_sample_topk on the device
    probs = logits_to_probs(logits[:, -1], temperature, top_k)
    return multinomial_sample_one_no_sync(probs), probs


# ------------------------------------------------------------------------------------------------
# generation
# ------------------------------------------------------------------------------------------------

@torch.no_grad()
def prefill(model, x: torch.Tensor, input_pos: torch.Tensor, **sampling_kwargs) -> torch.Tensor:
    logits = model(x, input_pos)
    return sample(logits, model=model, **sampling_kwargs)[0]


@torch.no_grad()
def decode_one_token(model, x: torch.Tensor, input_pos: torch.Tensor, **sampling_kwargs) -> Tuple[torch.Tensor, torch.Tensor]:
    assert input_pos.shape[-1] == 1
    logits = model(x, input_pos)
    return sample(logits, model=model, **sampling_kwargs)


@torch.no_grad()
def decode_n_tokens(model, cur_token: torch.Tensor, input_pos: torch.Tensor, num_new_tokens: int,
                    callback=lambda _: _, **sampling_kwargs):
    new_tokens, new_probs = [], []
    for _ in range(num_new_tokens):
        next_token, next_prob = decode_one_token(model, cur_token, input_pos, **sampling_kwargs)
        input_pos += 1
        new_tokens.append(next_token.clone())
        callback(new_tokens[-1])
        new_probs.append(None if next_prob is None else next_prob.clone())
        cur_token = new_tokens[-1]
    return new_tokens, new_probs


@torch.no_grad()
def generate(model, prompt: torch.Tensor, max_new_tokens: int, batch_size: int, empty: torch.Tensor, *,
             callback=lambda x: x, **sampling_kwargs):
    """Prefill the prompt (the same one in every batch row), then decode max_new_tokens - 1 steps.
    Returns (tokens [B, T + max_new_tokens], decode_latency, prefill_latency)."""
    T = prompt.size(-1)
    device = prompt.device
    rows = prompt.view(1, -1).repeat(batch_size, 1)
    empty[:, :T] = rows
    input_pos = torch.arange(0, T, device=device)

    device_sync(device)
    t0 = time.perf_counter()
    next_token = prefill(model, rows, input_pos, **sampling_kwargs)
    device_sync(device)
    prefill_latency = time.perf_counter() - t0
    print_rank_0(f"Prefill latency: {prefill_latency} sec")

    next_token = next_token.clone()
    empty[:, T] = next_token.squeeze(-1)
    input_pos = torch.tensor([T], device=device, dtype=torch.int)

    device_sync(device)
    t0 = time.perf_counter()
    generated, _ = decode_n_tokens(model, next_token.view(batch_size, -1), input_pos, max_new_tokens - 1,
                                   callback=callback, **sampling_kwargs)
    device_sync(device)
    decode_latency = time.perf_counter() - t0
    _raise_on_device_error(model)
    print_rank_0(f"Decode latency: {decode_latency} sec")
    if generated:
        empty[:, T + 1:] = torch.cat(generated, dim=-1)
    return empty, decode_latency, prefill_latency


def _raise_on_device_error(model):
    """After a synchronisation: a latency measured over steps that did no work (a position beyond the
    cache, an expired wait in the one-kernel step) must never be reported as a result."""
    check = getattr(model, "check_device_errors", None)
    if check is not None:
        check()


class DecodeGraph:
    """One decode step captured into a hipGraph: forward, next-token choice, and the device-side
    hand-over (token history write, cur_token <- next_token, pos += 1).  replay() is all a decode
    loop needs; the host never touches the static buffers between steps."""

    def __init__(self, model, batch_size: int, prompt_len: int, max_new_tokens: int, device, **sampling_kwargs):
        self.model, self.B, self.T = model, batch_size, prompt_len
        self.cur_token = torch.zeros(batch_size, 1, dtype=torch.int32, device=device)
        self.input_pos = torch.tensor([prompt_len], dtype=torch.int32, device=device)
        self.history = torch.zeros(batch_size, max(max_new_tokens - 1, 1), dtype=torch.int32, device=device)
        self.sampling_kwargs = sampling_kwargs

        def step():
            nxt, _ = decode_one_token(model, self.cur_token, self.input_pos, **sampling_kwargs)
            _hip.advance(self.cur_token, nxt.contiguous(), self.input_pos, batch_size, self.history, pos0=prompt_len)
            return nxt

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):  # warm-up outside capture (workspace allocation, lazy module loads)
                step()
        torch.cuda.current_stream().wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.next_token = step()

    def reset(self, first_token: torch.Tensor):
        self.cur_token.copy_(first_token.view(self.B, 1))
        self.input_pos.fill_(self.T)

    def replay(self):
        self.graph.replay()


@torch.no_grad()
def get_cuda_graphs_for_prefill(model, prompt: torch.Tensor, batch_size: int, **sampling_kwargs):
    T = prompt.size(-1)
    device = prompt.device
    static_x = prompt.view(1, -1).repeat(batch_size, 1)
    static_input_pos = torch.arange(0, T, device=device, dtype=torch.int32)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            prefill(model, static_x, static_input_pos, **sampling_kwargs)
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        static_next_token = prefill(model, static_x, static_input_pos, **sampling_kwargs)
    return g, static_x, static_input_pos, static_next_token


@torch.no_grad()
def get_cuda_graphs_for_decode(model, prompt: torch.Tensor, batch_size: int, max_new_tokens: int,
                               cur_token: torch.Tensor, **sampling_kwargs) -> DecodeGraph:
    dg = DecodeGraph(model, batch_size, prompt.size(-1), max_new_tokens, prompt.device, **sampling_kwargs)
    dg.reset(cur_token)
    return dg


@torch.no_grad()
def generate_using_cuda_graphs(prefill_graph, static_x, static_input_pos, static_next_token_prefill,
                               decode_graph: DecodeGraph, prompt: torch.Tensor, batch_size: int, empty: torch.Tensor,
                               num_new_tokens: int):
    T = prompt.size(-1)
    device = prompt.device
    rows = prompt.view(1, -1).repeat(batch_size, 1)
    empty[:, :T] = rows
    static_x.copy_(rows)

    device_sync(device)
    t0 = time.perf_counter()
    prefill_graph.replay()
    device_sync(device)
    prefill_latency = time.perf_counter() - t0
    print_rank_0(f"Prefill latency: {prefill_latency} sec")
    empty[:, T] = static_next_token_prefill.squeeze(-1)

    device_sync(device)
    t0 = time.perf_counter()
    decode_graph.reset(static_next_token_prefill)
    for _ in range(num_new_tokens - 1):
        decode_graph.replay()
    device_sync(device)
    decode_latency = time.perf_counter() - t0
    _raise_on_device_error(decode_graph.model)
    print_rank_0(f"Decode latency: {decode_latency} sec")
    if num_new_tokens > 1:
        empty[:, T + 1:] = decode_graph.history[:, : num_new_tokens - 1]
    return empty, decode_latency, prefill_latency


# ------------------------------------------------------------------------------------------------
# model construction
# ------------------------------------------------------------------------------------------------

def init_weights(model: torch.nn.Module, seed: Optional[int], std: float = 0.02):
    """N(0, std) for EVERY parameter, norm gains included, like the reference's _load_model; one
    seeded generator on the model's device, parameters visited in registration order."""
    params = list(model.parameters())
    gen = None
    if seed is not None and params:
        gen = torch.Generator(device=params[0].device)
        gen.manual_seed(seed)
    for p in params:
        torch.nn.init.normal_(p, mean=0.0, std=std, generator=gen)


def _load_model(model_name, device, precision, seed: Optional[int] = None, verbose: bool = True):
    family, config = model_name.split(":")
    with torch.device("meta"):
        model = _MODELS[family].from_name(config)
    model = model.to(dtype=precision)
    model = model.to_empty(device=device)
    with torch.no_grad():
        init_weights(model, seed)
    if verbose:
        print_rank_0(model)
    return model.eval()


def decode_bytes_per_step(cfg, batch_size: int, pos: int) -> int:
    """Algorithmic HBM bytes of one decode step at position `pos` (bf16): every weight and gain of
    the shard once, the valid K and V rows, the new K/V rows, the embedding rows."""
    D, L, hd = cfg.dim, cfg.n_layer, cfg.head_dim
    Hq, Hkv, I, V = cfg.n_head_local, cfg.n_kv_local, cfg.ffn_local, cfg.output_rows
    weights = L * (D * (Hq + 2 * Hkv) * hd + D * Hq * hd + D * 2 * I + I * D + 2 * D) + V * D + D
    kv_read = L * batch_size * 2 * Hkv * hd * (pos + 1)
    kv_write = L * batch_size * 2 * Hkv * hd
    emb = batch_size * D
    return 2 * (weights + kv_read + kv_write + emb)


# ------------------------------------------------------------------------------------------------
# main
# ------------------------------------------------------------------------------------------------

def main(model_name: str, prompt_length: int = 1, num_samples: int = 5, max_new_tokens: int = 100,
         batch_size: int = 1, top_k: int = 200, temperature: float = 0.8, compile: bool = True,
         compile_prefill: bool = False, profile: Optional[Path] = None, device=default_device,
         use_cuda_graphs: bool = False, greedy: bool = False, seed: Optional[int] = None,
         precision=torch.bfloat16, last_logits_only: bool = False, json_path: Optional[Path] = None,
         warmup: int = 5):
    from gpt_fast import maybe_init_dist

    rank = maybe_init_dist()
    if "cuda" not in str(device):
        raise RuntimeError("the HIP backend needs a GPU device; the CPU restatement lives in oracle/ (tests only)")
    _hip.load()
    print_rank_0(f"Using device={device}")
    print_rank_0("Loading model ...")
    t0 = time.time()
    model = _load_model(model_name, device, precision, seed)
    model.last_logits_only = last_logits_only
    device_sync(device)
    print_rank_0(f"Time to load model: {time.time() - t0:.02f} seconds")

    cfg = model.config
    gen = None
    if seed is not None:
        gen = torch.Generator(device=device)
        gen.manual_seed(seed + 1)
    hi = cfg.vocab_size if seed is not None else 1024  # the reference draws from [0, 1024)
    encoded = torch.randint(0, hi, (prompt_length,), device=device, dtype=torch.int64, generator=gen)
    torch.manual_seed(1234)
    model_size, params = _get_model_size(model)

    T_new = encoded.size(-1) + max_new_tokens
    max_seq_length = min(T_new, cfg.block_size)
    with torch.device(device):
        model.setup_caches(max_batch_size=batch_size, max_seq_length=max_seq_length)

    sampling = dict(temperature=temperature, top_k=top_k, greedy=greedy)
    graphs = compile or use_cuda_graphs
    if graphs:
        print_rank_0("hipGraph replay is active for decode" + (" and prefill" if compile_prefill or use_cuda_graphs
                                                               else ""))
        prefill_graph = None
        if compile_prefill or use_cuda_graphs:
            prefill_graph, static_x, static_input_pos, static_next_token_prefill = get_cuda_graphs_for_prefill(
                model, encoded, batch_size, **sampling)
        first = torch.zeros(batch_size, 1, dtype=torch.int32, device=device)
        decode_graph = get_cuda_graphs_for_decode(model, encoded, batch_size, max_new_tokens, first, **sampling)

    agg = {"tokens_per_sec_per_user": [], "total_tokens_per_sec": [], "decode_latency": [], "prefill_latency": []}
    start = 0 if profile else -warmup
    y = None
    for i in range(start, num_samples):
        device_sync(device)
        t0 = time.perf_counter()
        prof = contextlib.nullcontext()
        if profile and i == num_samples - 1:
            prof = torch.profiler.profile(
                activities=[torch.profiler.ProfilerActivity.CPU, torch.profiler.ProfilerActivity.CUDA],
                on_trace_ready=torch.profiler.tensorboard_trace_handler(str(profile)), record_shapes=True)
        empty = torch.empty(batch_size, T_new, dtype=encoded.dtype, device=device)
        with prof:
            if graphs and prefill_graph is not None:
                y, decode_latency, prefill_latency = generate_using_cuda_graphs(
                    prefill_graph, static_x, static_input_pos, static_next_token_prefill, decode_graph, encoded,
                    batch_size, empty, max_new_tokens)
            elif graphs:  # eager prefill, replayed decode
                T = encoded.size(-1)
                rows = encoded.view(1, -1).repeat(batch_size, 1)
                empty[:, :T] = rows
                device_sync(device)
                t1 = time.perf_counter()
                nxt = prefill(model, rows, torch.arange(0, T, device=device, dtype=torch.int32), **sampling).clone()
                device_sync(device)
                prefill_latency = time.perf_counter() - t1
                print_rank_0(f"Prefill latency: {prefill_latency} sec")
                empty[:, T] = nxt.squeeze(-1)
                t1 = time.perf_counter()
                decode_graph.reset(nxt)
                for _ in range(max_new_tokens - 1):
                    decode_graph.replay()
                device_sync(device)
                decode_latency = time.perf_counter() - t1
                _raise_on_device_error(model)
                print_rank_0(f"Decode latency: {decode_latency} sec")
                if max_new_tokens > 1:
                    empty[:, T + 1:] = decode_graph.history[:, : max_new_tokens - 1]
                y = empty
            else:
                y, decode_latency, prefill_latency = generate(model, encoded, max_new_tokens, batch_size=batch_size,
                                                              empty=empty, **sampling)
        if i == start and start < 0:
            print_rank_0(f"Compilation time: {time.perf_counter() - t0:.2f} seconds")
        device_sync(device)
        if i < 0:
            continue
        t = time.perf_counter() - t0
        per_user = (y.size(-1) - prompt_length) / t
        total = per_user * y.size(0)
        agg["tokens_per_sec_per_user"].append(per_user)
        agg["total_tokens_per_sec"].append(total)
        agg["decode_latency"].append(decode_latency)
        agg["prefill_latency"].append(prefill_latency)
        print_rank_0(f"Time for inference {i + 1}: {t:.02f} sec total")
        print_rank_0(f"Tokens per second per user: {per_user:.02f} tokens/sec/user")
        print_rank_0(f"Total tokens per second: {total:.02f} tokens/sec")
        print_rank_0(f"Decode latency: {decode_latency:.02f} sec")
        print_rank_0(f"Prefill latency: {prefill_latency:.02f} sec")
        print_rank_0(f"Bandwidth achieved: {model_size * per_user / 1e9:.02f} GB/s")
        print_rank_0(f"FLOPS achieved: {params * (y.numel() / t) * 2 / 1e12:.02f} TF/s")
        print_rank_0()

    mean = lambda k: float(torch.tensor(agg[k]).mean())
    steps = max(max_new_tokens - 1, 1)
    ms_per_token = mean("decode_latency") / steps * 1e3
    mid_pos = prompt_length + steps // 2
    step_bytes = decode_bytes_per_step(cfg, batch_size, mid_pos)
    gbps = step_bytes / (ms_per_token * 1e-3) / 1e9
    print_rank_0("==========")
    print_rank_0(f"Batch Size: {batch_size}")
    print_rank_0(f"Prompt Length: {prompt_length}")
    print_rank_0(f"Generated tokens: {max_new_tokens}")
    print_rank_0(f"Average decode latency: {mean('decode_latency'):.04f} sec")
    print_rank_0(f"Average prefill latency: {mean('prefill_latency'):.04f} sec")
    print_rank_0(f"Average tokens/sec/user: {mean('tokens_per_sec_per_user'):.2f}")
    print_rank_0(f"Average tokens/sec: {mean('total_tokens_per_sec'):.2f}")
    print_rank_0(f"Decode: {ms_per_token:.3f} ms/token, {batch_size * 1e3 / ms_per_token:.1f} tok/s, "
                 f"{gbps:.0f} GB/s algorithmic = {100 * gbps / HBM_PEAK_GBPS:.1f} % of {HBM_PEAK_GBPS:.0f} GB/s")
    print_rank_0(f"Memory used: {torch.cuda.max_memory_reserved() / 1e9:.02f} GB")
    result = dict(model_name=model_name, batch_size=batch_size, prompt_length=prompt_length,
                  max_new_tokens=max_new_tokens, ms_per_token=ms_per_token,
                  decode_tok_per_s=batch_size * 1e3 / ms_per_token, prefill_latency_s=mean("prefill_latency"),
                  decode_latency_s=mean("decode_latency"), algorithmic_bytes_per_step=step_bytes,
                  achieved_GBps=gbps, roofline_fraction=gbps / HBM_PEAK_GBPS,
                  tokens=y[0, prompt_length:].tolist() if y is not None else [])
    if json_path:
        Path(json_path).write_text(json.dumps(result))
    print_rank_0("Done.")
    return result


def build_parser():
    p = argparse.ArgumentParser(description="Per-rank Ladder-Residual inference benchmark on MI355X (HIP backend).")
    p.add_argument("--model_name", type=str, required=True, help="family:config, e.g. gpt_ladder:ladder-70b-tp8")
    p.add_argument("--prompt_length", type=int, required=True, help="Input prompt length")
    p.add_argument("--num_samples", type=int, default=5, help="Number of samples.")
    p.add_argument("--max_new_tokens", type=int, default=200, help="Maximum number of new tokens.")
    p.add_argument("--batch_size", type=int, default=1, help="Batch size to benchmark with")
    p.add_argument("--top_k", type=int, default=200, help="Top-k for sampling.")
    p.add_argument("--temperature", type=float, default=0.8, help="Temperature for sampling.")
    p.add_argument("--compile", action="store_true", help="Replay the decode step as a hipGraph.")
    p.add_argument("--compile_prefill", action="store_true", help="Also replay prefill as a hipGraph.")
    p.add_argument("--cuda_graph", action="store_true", help="Capture prefill and decode into hipGraphs.")
    p.add_argument("--use_flash_attention", action="store_true", help="Accepted; the HIP attention path is unchanged.")
    p.add_argument("--profile", type=Path, default=None, help="Profile path.")
    p.add_argument("--device", type=str, default=default_device, help="Device to use")
    p.add_argument("--greedy", action="store_true", help="argmax decoding (lowest index on ties)")
    p.add_argument("--seed", type=int, default=None, help="seed for weights and prompt")
    p.add_argument("--virtual_tp", type=int, default=None, help="build layers as one rank of this many")
    p.add_argument("--tp_rank", type=int, default=0)
    p.add_argument("--shard_vocab", action="store_true",
                   help="with --virtual_tp: the lm_head keeps vocab_size / virtual_tp rows as well")
    p.add_argument("--last_logits_only", action="store_true", help="prefill computes logits of the last position only")
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--json", type=Path, default=None, help="write the summary here")
    return p


if __name__ == "__main__":
    args = build_parser().parse_args()
    if args.cuda_graph:
        assert not args.compile
    if args.shard_vocab and not args.virtual_tp:
        raise SystemExit("--shard_vocab needs --virtual_tp")
    if args.virtual_tp:
        set_virtual_tp(args.virtual_tp, args.tp_rank, args.shard_vocab)
    print_rank_0(f"flash_kv_decode is set to {args.use_flash_attention}")
    with set_flash_attention(args.use_flash_attention):
        main(args.model_name, args.prompt_length, args.num_samples, args.max_new_tokens, args.batch_size, args.top_k,
             args.temperature, args.compile, args.compile_prefill, args.profile, args.device, args.cuda_graph,
             greedy=args.greedy, seed=args.seed, last_logits_only=args.last_logits_only, json_path=args.json,
             warmup=args.warmup)
