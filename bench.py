"""Decode and prefill throughput of the Qwen3-4B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]
    python bench.py --workload qwen3-8b-mixed | qwen3-32b-decode     (two further workloads)
    python bench.py --generate                                       (the decode workload through LLM.generate)
    python bench.py --workload gufasun [--shape 4b|8b] [--layers L]  (the Gufasun design beside Qwen3 at equal sizes)
    python bench.py --workload sovutar [--shape 4b|8b] [--layers L]  (the Sovutar design beside Qwen3 at equal sizes)
    python bench.py --workload tazitar [--shape 4b|8b] [--layers L]  (the Tazitar design beside Qwen3 at equal sizes)
    python bench.py --workload retudra [--shape 4b|8b] [--layers L]  (the Retudra design beside Sovutar and Qwen3 at equal sizes)

A step is one decode step of `batch` requests, each holding a `prompt`-token random prompt
(prefilled by the engine itself before the clock starts) and growing by one token per step.
`value` is decoded tokens per second over exactly K timed steps.  The same line carries the
prefill of one 2,048-token prompt, the decode step's HBM roofline, and decode at batch 1 and 64.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# the benchmark configuration: Qwen3-4B shape
QWEN3_4B = dict(num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
                head_dim=128, intermediate_size=9728, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=40960)
# the two further workloads (`--workload`): Qwen3-8B and Qwen3-32B shapes
QWEN3_8B = dict(num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960)
QWEN3_32B = dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                 head_dim=128, intermediate_size=25600, vocab_size=151936, rope_theta=1000000.0,
                 rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960)
FULL_LAYERS = QWEN3_4B["num_hidden_layers"]
CONTEXT = 4096
PROMPT = 2048
PAGE = 16


def layer_params(c) -> int:
    q, kv = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    h, i = c["hidden_size"], c["intermediate_size"]
    return h * (q + 2 * kv) + q * h + 3 * h * i


def decode_bytes(c, batch: int, context: float, elt: int = 2) -> float:
    """Bytes one decode step has to read: every weight once and the cache of the live requests."""
    L, h = c["num_hidden_layers"], c["hidden_size"]
    weights = (L * (layer_params(c) + 2 * h + 2 * c["head_dim"]) + h + c["vocab_size"] * h) * elt
    kv = batch * context * 2 * L * c["num_key_value_heads"] * c["head_dim"] * elt
    return weights + kv


def prefill_flops(c, tokens: int) -> float:
    L = c["num_hidden_layers"]
    gemm = 2.0 * tokens * L * layer_params(c)
    attn = 4.0 * c["num_attention_heads"] * c["head_dim"] * (tokens * (tokens + 1) / 2) * L
    head = 2.0 * c["vocab_size"] * c["hidden_size"]
    return gemm + attn + head


# ---- where a step's time goes: kernels of a profiled step, sorted into the parts of a layer -------------------------

GEMM_NAMES = ("gemm_rows", "gemm_stream", "gemm_tiles", "gemm_f32", "Cijk_", "sum_partials", "silu_mul")
PARTS = ("qkv", "o", "gate_up", "down", "head", "attention", "qk_prep", "norm", "other")


def _template_args(name: str) -> list:
    return name[name.index("<") + 1:name.rindex(">")].replace(" ", "").split(",") if "<" in name and ">" in name else []


def _completes_gate_up(name: str) -> bool:
    """Whether this kernel leaves gate|up complete: a product with the activation fused (gemm_rows_kernel<MT, WN,
    WK, PD, XD, EPI, out> / gemm_tiles_kernel<MT, TN, PD, PX, PIPE, EPI, out> with EPI = 1), or the activation kernel
    behind a plain product."""
    if "silu_mul" in name:
        return True
    args = _template_args(name)
    if "gemm_rows_kernel" in name:
        return len(args) > 5 and args[5] == "1"
    if "gemm_tiles_kernel" in name:
        return len(args) > 5 and args[5] == "1"
    return False


def classify_step(names, layers: int) -> list:
    """The part of the model that each kernel of one step belongs to, from the order in which a layer launches
    them: norm, q|k|v product, q/k preparation (a kernel of its own, or inside the attention's for single decoded
    tokens), attention (+ merges), o product, norm, gate|up (+ activation), down product; after the last layer the
    final norm and the head."""
    out, phase, layers_done = [], "qkv", 0
    for name in names:
        if "qk_prep" in name:
            part, phase = "qk_prep", "o"
        elif "attn_" in name:
            part = "attention"
            if phase == "qkv":     # single decoded tokens: the attention's kernel prepares q, k and v itself
                phase = "o"
        elif "rmsnorm" in name:
            part = "norm"
            if phase == "o":
                phase = "gate_up"
            elif phase == "down":
                layers_done += 1
                phase = "head" if layers_done >= layers else "qkv"
        elif any(g in name for g in GEMM_NAMES):
            part = phase
            if phase == "gate_up" and _completes_gate_up(name):
                phase = "down"
        else:
            part = "other"
        out.append(part)
    return out


def profiled_steps(torch, fns) -> list:
    """The kernels of every call in `fns`, run one after the other inside ONE profiler session (a second session
    in a process has crashed the profiler here): a list, one entry a call, of (name, microseconds) in launch
    order.  A step begins with the embedding kernel, which is how the session's kernels are cut into calls."""
    from torch.profiler import ProfilerActivity, profile

    torch.cuda.synchronize()
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        for fn in fns:
            fn()
            torch.cuda.synchronize()
    evs = [e for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA and "Memcpy" not in e.name
           and "Memset" not in e.name]
    evs.sort(key=lambda e: e.time_range.start)
    steps, early = [], []
    for e in evs:
        item = (e.name, e.time_range.end - e.time_range.start)
        if "embed_gather" in e.name:
            steps.append(early + [item])     # what ran before the first step's embedding is counted with it
            early = []
        elif steps:
            steps[-1].append(item)
        else:
            early.append(item)
    if len(steps) != len(fns):
        raise RuntimeError(f"the profiler saw {len(steps)} steps for {len(fns)} calls")
    return steps


def part_times(steps, layers: int) -> dict:
    """part -> microseconds a step (mean over `steps`, lists of (kernel name, microseconds)), plus "kernels".
    The profiler now and then loses kernels of a step; only the steps with the most kernels are counted, and
    those must show every layer."""
    most = max(len(k) for k in steps)
    steps = [k for k in steps if len(k) == most]
    for kernels in steps:
        seen = (sum(1 for n, _ in kernels if "rmsnorm" in n) - 1) // 2   # two norms a layer and the last one
        if seen != layers:
            raise RuntimeError(f"a profiled step shows {seen} of {layers} layers")
    total = {p: 0.0 for p in PARTS}
    for kernels in steps:
        for part, (_, us) in zip(classify_step([n for n, _ in kernels], layers), kernels):
            total[part] += us
    out = {p: t / len(steps) for p, t in total.items()}
    missing = [p for p in ("qkv", "o", "gate_up", "down", "head") if not out.get(p)]
    if missing:  # a kernel's name no longer says what the sorting reads from it
        raise RuntimeError(f"no kernel of a profiled step was sorted into {', '.join(missing)}")
    out["kernels"] = sum(len(k) for k in steps) / len(steps)
    return out


def part_bytes_decode(c, batch: int, context: float, elt: int = 2) -> dict:
    """Bytes that each part of a decode step has to read: its weights once, and for attention the cache."""
    L, h, i = c["num_hidden_layers"], c["hidden_size"], c["intermediate_size"]
    q, kv = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    return {"qkv": L * h * (q + 2 * kv) * elt, "o": L * q * h * elt, "gate_up": L * 2 * i * h * elt,
            "down": L * h * i * elt, "head": c["vocab_size"] * h * elt, "attention": batch * context * 2 * L * kv * elt}


def part_flops_prefill(c, tokens: int) -> dict:
    L, h, i = c["num_hidden_layers"], c["hidden_size"], c["intermediate_size"]
    q, kv = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    return {"qkv": 2.0 * tokens * L * h * (q + 2 * kv), "o": 2.0 * tokens * L * q * h,
            "gate_up": 2.0 * tokens * L * 2 * i * h, "down": 2.0 * tokens * L * h * i,
            "head": 2.0 * c["vocab_size"] * h, "attention": 4.0 * q * (tokens * (tokens + 1) / 2) * L}


def part_report(times: dict, work: dict, peak: float, ceiling: float) -> tuple:
    """(microseconds a step by part, fraction of the published peak, fraction of the measured ceiling)."""
    us = {p: round(times[p], 1) for p in PARTS if times.get(p)}
    us["kernels"] = round(times["kernels"], 1)
    of_peak = {p: round(work[p] / (times[p] * 1e-6) / peak, 4) for p in work if times.get(p)}
    of_ceiling = {p: round(work[p] / (times[p] * 1e-6) / ceiling, 4) for p in work if times.get(p)}
    return us, of_peak, of_ceiling


def parts_in_a_child_process(args) -> dict:
    """The breakdown by part of the model, measured by a second run of this program under the profiler: the
    profiler stays out of the process whose steps are timed, and a fault of its own costs only the breakdown."""
    import os
    import subprocess

    cmd = [sys.executable, os.path.abspath(__file__), "--parts-only", "--batch", str(args.batch), "--layers", str(args.layers),
           "--page-size", str(PAGE), "--dtype", args.dtype]
    cmd += ["--no-weight-tiles"] if args.no_weight_tiles else []
    try:
        res = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        lines = [ln for ln in res.stdout.splitlines() if ln.startswith("{")]
        if res.returncode != 0 or not lines:
            return {"parts": f"not measured: the profiled run ended with code {res.returncode}"}
        return json.loads(lines[-1])
    except (subprocess.TimeoutExpired, OSError, ValueError) as exc:
        return {"parts": f"not measured: {type(exc).__name__}"}


def _timed(torch, fn):
    torch.cuda.synchronize()
    t = time.perf_counter()
    fn()
    torch.cuda.synchronize()
    return time.perf_counter() - t


def ceilings() -> int:
    """What a kernel that only reads memory and one that only multiplies reach on this GPU, against the published peaks."""
    import torch

    from arle_amd.kernels import ceilings as c

    read = c.read_bandwidth()
    small = c.read_bandwidth(launches=40)
    m32, m16 = c.mfma_rate(shape=32), c.mfma_rate(shape=16)
    same32 = c.mfma_rate(shape=32, random_operands=False)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    # one workgroup of four waves a busy compute unit: what a product costs in time says what the clock is (32 cycles)
    by_busy = {n: c.mfma_rate(shape=32, workgroups=n, repeats=2) for n in (cus // 8, cus // 2, 3 * cus // 4, cus)}
    print(json.dumps({
        "metric": "measured ceilings of one GPU", "unit": "GB/s and TFLOP/s",
        "hbm_read_gbs": round(read["best"] / 1e9, 1), "hbm_read_frac_of_peak": round(read["best"] / 1e9 / PEAK_HBM_GBS, 4),
        "hbm_read_100mb_launches_gbs": round(small["best"] / 1e9, 1),
        "hbm_read_by_workgroups_gbs": {str(k): round(v / 1e9, 1) for k, v in read["by_workgroups"].items()},
        "mfma_bf16_32x32x16_tflops": round(m32 / 1e12, 1), "mfma_bf16_16x16x32_tflops": round(m16 / 1e12, 1),
        "mfma_frac_of_peak": round(max(m32, m16) / PEAK_FLOPS["bf16"], 4),
        "mfma_bf16_32x32x16_same_operands_tflops": round(same32 / 1e12, 1),
        "mfma_clock_ghz_by_busy_cus": {str(n): round(v / (n * 4 * 32768.0 / 32.0) / 1e9, 2) for n, v in by_busy.items()}}))
    return 0


def mixed_8b(args) -> int:
    """Qwen3-8B shape: 32 requests decoding at 1,024 tokens of context beside one 2,048-token prompt
    that arrives in portions of 512, cut as the scheduler cuts them (aligned_portion: four steps of 32 + 512
    rows, since stopping at 480 would cost this prompt a fifth step).  Every step is launched from the last one's
    tokens on the GPU; --no-overlap: each waits for its tokens on the host.
    Reports the mean step and the tokens a second of both kinds."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.engine.scheduler import SchedulerConfig, aligned_portion
    from arle_amd.kernels import ops
    from arle_amd.sampling import Sampler, SamplingParams

    raw = dict(QWEN3_8B, num_hidden_layers=args.layers or QWEN3_8B["num_hidden_layers"])
    config = Qwen3Config.from_dict(raw)
    decoders, context, prompt, portion = 32, 1024, 2048, 512
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=decoders * (context + 64) + 2 * prompt, max_slots=decoders + 1,
                                max_request_tokens=4096)
    gen = torch.Generator().manual_seed(1234)
    rand = lambda n: torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()
    keys = [("d", i) for i in range(decoders)]
    last = []
    for k in keys:
        engine.add_request(k)
    for i in range(0, decoders, 8):
        out = engine.step([StepEntry(k, rand(context - 1), [context - 2]) for k in keys[i:i + 8]])
        last.extend(ops.argmax_rows(out).tolist())
    state = {"last": last, "chosen": None}
    sampler = Sampler(engine.device)
    greedy = [(SamplingParams(), 0, 0, [])] * (decoders + 1)
    align = 0 if args.no_overlap else SchedulerConfig().step_row_alignment
    cuts, a = [], 0
    while a < prompt:       # the portions as Scheduler.plan_prefill cuts them
        n = aligned_portion(min(prompt - a, portion), prompt - a, decoders, align)
        cuts.append((a, n))
        a += n

    def one_prompt(tag):
        engine.add_request(tag)
        toks = rand(prompt)
        for a, n in cuts:
            before = state["chosen"]
            if before is None:
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
            else:
                entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
            last_piece = a + n == prompt
            entries.append(StepEntry(tag, toks[a:a + n], [n - 1] if last_piece else []))
            chosen = sampler.choose(engine.step(entries, borrow_logits=True), greedy[:decoders + (1 if last_piece else 0)])
            if args.no_overlap:
                state["last"] = chosen.tokens()[:decoders]
            else:
                state["chosen"] = chosen
                if before is not None:
                    state["last"] = before.tokens()[:decoders]
        engine.end_request(tag)

    def settle():
        if state["chosen"] is not None:
            state["last"], state["chosen"] = state["chosen"].tokens()[:decoders], None

    for i in range(2):          # the second pass captures the step shapes, later ones replay them
        one_prompt(("warm", i))
    settle()
    # the decoders have grown by a few tokens; the timed prompts run just above 1,024 tokens of context
    reps = max(1, args.steps // len(cuts))
    dt = _timed(torch, lambda: ([one_prompt(("p", i)) for i in range(reps)], settle()))
    steps = len(cuts) * reps
    ms = dt / steps * 1e3
    flops = sum(prefill_flops_portion(raw, a, n) for a, n in cuts) / len(cuts)
    portion = prompt / len(cuts)     # mean tokens of a portion
    line = {"metric": "mixed step: 32 decoding requests at 1,024 tokens + a 512-token prompt portion (Qwen3-8B shape)",
            "value": round(steps * (decoders + portion) / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps,
            "warmup": 8, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic: seeded random weights N(0,0.02), uniform random token ids",
            "config": {"model": "Qwen3-8B shape", "decoding_requests": decoders, "decode_context": context,
                       "prompt_len": prompt, "portions": " ".join(str(n) for _, n in cuts), "layers": raw["num_hidden_layers"],
                       "hidden": raw["hidden_size"], "q_heads": 32, "kv_heads": 8, "head_dim": 128,
                       "intermediate": raw["intermediate_size"], "vocab": raw["vocab_size"], "tied": False,
                       "page_size": PAGE},
            "points": {"decode_tok_s": round(decoders * steps / dt, 1), "prefill_tok_s": round(portion * steps / dt, 1)},
            "roofline": {"bound": "mfma+hbm", "flops_per_step": round(flops / 1e12, 2), "unit": "TFLOP",
                         "frac": round(flops / (dt / steps) / PEAK_FLOPS["bf16"], 4)}}
    print(json.dumps(line))
    return 0


def prefill_flops_portion(c, start: int, n: int) -> float:
    """Flops of a portion of n prompt tokens that starts at position `start` (products and causal attention)."""
    L = c["num_hidden_layers"]
    gemm = 2.0 * n * L * layer_params(c)
    attn = 4.0 * c["num_attention_heads"] * c["head_dim"] * (n * start + n * (n + 1) / 2) * L
    return gemm + attn


def decode_32b(args) -> int:
    """Qwen3-32B shape: 64 requests decoding at 8,192 tokens of context by default (65 GB of
    weights, 137 GB of cache)."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops

    raw = dict(QWEN3_32B, num_hidden_layers=args.layers or QWEN3_32B["num_hidden_layers"])
    config = Qwen3Config.from_dict(raw)
    batch, context = args.batch or 64, args.context
    steps, warmup = min(args.steps, 16), min(args.warmup, 4)
    t0 = time.time()
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=batch * (context + 64), max_slots=batch, max_request_tokens=context + 64)
    print(f"[bench] engine ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(1234)
    rand = lambda n: torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()
    keys = [("d", i) for i in range(batch)]
    last = []
    for i, k in enumerate(keys):          # real prefill, one 8,191-token prompt a step
        engine.add_request(k)
        out = engine.step([StepEntry(k, rand(context - 1), [context - 2])])
        last.extend(ops.argmax_rows(out).tolist())
        if i % 8 == 7:
            print(f"[bench] prefilled {i + 1} of {batch} requests ({time.time() - t0:.0f} s)", file=sys.stderr, flush=True)
    state = {"last": last, "chosen": None}
    from arle_amd.sampling import Sampler, SamplingParams
    sampler, greedy = Sampler(engine.device), [(SamplingParams(), 0, 0, [])] * batch

    def one_step():     # launched from the last step's tokens on the GPU, those read meanwhile; --no-overlap: waiting
        before = state["chosen"]
        if before is None:
            entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
        else:
            entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
        chosen = sampler.choose(engine.step(entries, borrow_logits=True), greedy)
        if args.no_overlap:
            state["last"] = chosen.tokens()
        else:
            state["chosen"] = chosen
            if before is not None:
                state["last"] = before.tokens()

    def settle():
        if state["chosen"] is not None:
            state["last"], state["chosen"] = state["chosen"].tokens(), None

    for _ in range(warmup):
        one_step()
    settle()
    ctx0 = engine.length(keys[0])
    dt = _timed(torch, lambda: ([one_step() for _ in range(steps)], settle()))
    ctx_mean = ctx0 + (steps - 1) / 2.0 + 1
    achieved = decode_bytes(raw, batch, ctx_mean) / (dt / steps) / 1e9
    line = {"metric": f"decode tok/s at batch {batch}, {context:,} tokens of context (Qwen3-32B shape, random weights)",
            "value": round(batch * steps / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(dt / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic: seeded random weights N(0,0.02), uniform random token ids",
            "config": {"model": "Qwen3-32B shape", "global_batch": batch, "seq_len": context, "layers": raw["num_hidden_layers"],
                       "layers_full": QWEN3_32B["num_hidden_layers"], "hidden": raw["hidden_size"], "q_heads": 64,
                       "kv_heads": 8, "head_dim": 128, "intermediate": raw["intermediate_size"],
                       "vocab": raw["vocab_size"], "tied": False, "page_size": PAGE},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(achieved / PEAK_HBM_GBS, 4)}}
    print(json.dumps(line))
    return 0


def step_gaps(args) -> int:
    """Decode steps of the Qwen3-4B shape both ways, steps that wait for their tokens on the host and steps launched
    from the last one's tokens on the GPU: milliseconds a step, and from a kernel timeline of six steps how long
    the GPU works and how long it idles between kernels in a step.  One JSON line a batch size."""
    import torch
    from torch.profiler import ProfilerActivity, profile

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops
    from arle_amd.sampling import Sampler, SamplingParams

    raw = dict(QWEN3_4B, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    batches = [args.batch] if args.batch else [1, 8, 64]
    most = max(batches)
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=most * (PROMPT + 256), max_slots=most, max_request_tokens=PROMPT + 256)
    sampler = Sampler(engine.device)
    gen = torch.Generator().manual_seed(1234)
    for batch in batches:
        keys, last = [("g", batch, i) for i in range(batch)], []
        rows = [(SamplingParams(), 0, 0, [])] * batch
        for k in keys:
            engine.add_request(k)
            toks = torch.randint(0, config.vocab_size, (PROMPT,), generator=gen).tolist()
            last.append(int(ops.argmax_rows(engine.step([StepEntry(k, toks, [PROMPT - 1])]))[0]))
        state = {"last": last, "chosen": None}

        def waiting():
            out = engine.step([StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])])
            state["last"] = sampler.choose(out, rows).tokens()

        def ahead():
            before = state["chosen"]
            if before is None:
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
            else:
                entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
            state["chosen"] = sampler.choose(engine.step(entries, borrow_logits=True), rows)
            if before is not None:
                state["last"] = before.tokens()

        def settle():
            if state["chosen"] is not None:
                state["last"], state["chosen"] = state["chosen"].tokens(), None

        line = {"metric": f"decode step at batch {batch}, {PROMPT}-token prompts (Qwen3-4B shape): steps that wait "
                          f"for their tokens and steps launched ahead", "unit": "ms a step", "n_gpus": 1, "dtype": "bf16",
                "layers": args.layers}
        for name, fn in (("waiting", waiting), ("ahead", ahead)):
            for _ in range(8):
                fn()
            settle()
            wall = _timed(torch, lambda: ([fn() for _ in range(args.steps)], settle())) / args.steps
            with profile(activities=[ProfilerActivity.CUDA]) as prof:
                for _ in range(7):
                    fn()
                settle()
                torch.cuda.synchronize()
            evs = sorted((e for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA),
                         key=lambda e: e.time_range.start)
            first = [i for i, e in enumerate(evs) if "embed_gather" in e.name]
            evs = evs[first[1]:first[-1]]          # whole steps 2..6: the first carries the profiler's start
            n = len(first) - 2
            busy = sum(e.time_range.end - e.time_range.start for e in evs) / n
            span = (evs[-1].time_range.end - evs[0].time_range.start) / n
            line[name] = {"ms_per_step": round(wall * 1e3, 4), "gpu_busy_us": round(busy, 1), "gpu_idle_us": round(span - busy, 1),
                          "kernels": round(len(evs) / n, 1)}
        print(json.dumps(line), flush=True)
        for k in keys:
            engine.end_request(k)
    return 0


def first_token(args) -> int:
    """Time to the first token through `LLM.generate` (scheduler, sampler, engine) for one prompt of 2,048, 8,192 and
    16,000 tokens and for four prompts of 2,048 at once, with the portion size that the GPU's memory gives (the
    default) and with portions of 512: one JSON line each."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine
    from arle_amd.engine.api import LLM

    raw = dict(QWEN3_4B, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    longest = 16384 + 64
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=4 * longest, max_slots=4, max_request_tokens=longest)
    gen = torch.Generator().manual_seed(1234)
    rand = lambda n: torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()
    for chunk in (None, 512):
        llm = LLM(engine, num_slots=4, chunked_prefill_size=chunk, max_seq_len=longest)
        for prompts in ([2048], [8192], [16000], [2048] * 4):
            batch = [rand(n) for n in prompts]
            for _ in range(3):      # the third run replays what the first two captured
                outs = llm.generate(batch, max_tokens=4, ignore_eos=True)
            ttft = max(o.ttft_s for o in outs)
            print(json.dumps({"metric": f"time to the first token of {len(prompts)} prompt(s) of {prompts[0]:,} tokens "
                                        f"through LLM.generate (Qwen3-4B shape)", "value": round(ttft * 1e3, 2), "unit": "ms",
                              "higher_is_better": False, "n_gpus": 1, "dtype": "bf16", "layers": args.layers,
                              "chunked_prefill_size": llm.sched_config.chunked_prefill_size,
                              "prefill_steps": llm.last_stats["steps"]["prefill"],
                              "prompt_tok_s": round(sum(prompts) / ttft, 1)}), flush=True)
    return 0


def generate_workload(args) -> int:
    """The decode workload of the baseline's benchmark configuration as a user runs it: 1, 8 and 64 prompts of 2,048
    uniform-random tokens, 256 tokens generated for each, through `LLM.generate` (scheduler, sampler, engine; greedy
    and at temperature 0.8).  One JSON line each: generated tokens a second after the first token, the time to the
    first token of the last prompt served, and the steps by kind."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine
    from arle_amd.engine.api import LLM

    config = Qwen3Config.from_dict(dict(QWEN3_4B, num_hidden_layers=args.layers))
    prompt, new, most = args.prompt_len, 256, 64
    longest = -(-(prompt + new + 1) // 64) * 64
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=args.page_size,
                                max_tokens=most * longest, max_slots=most, max_request_tokens=longest)
    gen = torch.Generator().manual_seed(1234)
    for temperature in (0.0, 0.8):
        for n in (1, 8, most):
            llm = LLM(engine, num_slots=most, max_seq_len=longest)
            prompts = [torch.randint(0, config.vocab_size, (prompt,), generator=gen).tolist() for _ in range(n)]
            for _ in range(3):      # the third run replays what the first two captured (a shape is captured when it repeats)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                outs = llm.generate(prompts, max_tokens=new, temperature=temperature, seed=3, ignore_eos=True)
                torch.cuda.synchronize()
                wall = time.perf_counter() - t0
            ttft = max(o.ttft_s for o in outs)
            made = sum(o.usage.completion_tokens for o in outs)
            print(json.dumps({"metric": f"{n} prompt(s) of {prompt:,} tokens, {new} generated each, through LLM.generate "
                                        f"(Qwen3-4B shape, temperature {temperature})",
                              "value": round((made - n) / (wall - ttft), 1), "unit": "generated tok/s after the first token",
                              "higher_is_better": True, "n_gpus": 1, "dtype": "bf16", "layers": args.layers,
                              "wall_s": round(wall, 4), "ttft_ms": round(ttft * 1e3, 1),
                              "ms_per_token_a_request": round(sum(o.tpot_s for o in outs) / n * 1e3, 3),
                              "steps": llm.last_stats["steps"]}), flush=True)
    return 0


def tune_products(args) -> int:
    """Measure the table of `arle_amd.kernels.tune` for one model's widths and write it; one line a (product, row
    count) to stderr, and at the end what the table gains over the rules at every row count where they differ."""
    from arle_amd.kernels import tune

    named = {"4b": (2560, 4096, 1024, 9728, 151936), "8b": (4096, 4096, 1024, 12288, 151936),
             "32b": (5120, 8192, 1024, 25600, 151936)}
    widths = named.get(args.tune_products) or tuple(int(v) for v in args.tune_products.split(","))
    if len(widths) not in (4, 5):
        print("--tune-products takes 4b, 8b, 32b or hidden,q_width,kv_width,intermediate[,vocabulary]", file=sys.stderr)
        return 2

    def say(rec):
        print(f"[tune] {rec['product']:8s} rows {rec['rows']:5d}: rule {rec['rule'][0]:13s} {rec['rule_us']:8.1f} us   "
              f"best {rec['best'][0]:13s} {rec['best_us']:8.1f} us", file=sys.stderr, flush=True)

    table, report = tune.tune_products(tune.model_products(*widths), tiled=not args.no_weight_tiles, say=say)
    path = args.out or f"product_table_{args.tune_products.replace(',', '_')}.json"
    if os.path.exists(path):       # a file may hold the tables of several runs (with and without operand tiles)
        with open(path, encoding="utf-8") as fh:
            table = {**json.load(fh), **table}
    tune.write_table(path, table)
    changed = [r for r in report if r["best"] != r["rule"]]
    print(json.dumps({"table": path, "points": len(report), "points_where_the_table_differs": len(changed),
                      "gain_us": {f"{r['product']}@{r['rows']}": round(r["rule_us"] - r["best_us"], 1) for r in changed}}))
    return 0


def sweep(args) -> int:
    """Further sizes of the Qwen3-4B shape, one JSON line each with its fraction of the roofline: decode at batch 16
    and 32 (2,048-token prompts), at batch 128 and 256 (1,024 tokens of context), at batch 8 with 8,192, 16,384 and
    32,768 tokens of context, at batch 64 with 16,384, prefills of 32,768, 16,384, 8,192, 512 and 128 tokens, and a
    504-token prompt portion beside 8 decoding requests."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops

    raw = dict(QWEN3_4B, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    longest = 32768 + args.steps + 16     # the longest context, its warm-up and timed steps
    most_tokens = max(8 * longest + 40 * 4096, 64 * (16384 + args.steps + 16), 256 * (1024 + args.steps + 16))
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=most_tokens, max_slots=257, max_request_tokens=longest)
    gen = torch.Generator().manual_seed(1234)
    rand = lambda n: torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()
    from arle_amd.sampling import Sampler, SamplingParams
    sampler, greedy_rows = Sampler(engine.device), [(SamplingParams(), 0, 0, [])] * 257
    base = {"n_gpus": 1, "dtype": "bf16", "higher_is_better": True, "data": "synthetic", "layers": args.layers}

    def fill(keys, context, portion=8192):
        last = []
        for k in keys:
            engine.add_request(k)
            toks = rand(context)
            for a in range(0, context, portion):
                piece = toks[a:a + portion]
                out = engine.step([StepEntry(k, piece, [len(piece) - 1] if a + portion >= context else [])])
            last.append(int(ops.argmax_rows(out)[0]))
        return last

    def decode_point(batch, context, steps):
        keys = [("s", batch, context, i) for i in range(batch)]
        state = {"last": fill(keys, context)}

        def one_step():     # as the headline run: launched from the last step's tokens on the GPU, those read meanwhile
            before = state.get("chosen")
            if before is None:
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
            else:
                entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
            state["chosen"] = sampler.choose(engine.step(entries, borrow_logits=True), greedy_rows[:batch])
            if before is not None:
                state["last"] = before.tokens()

        def settle():
            state["last"] = state.pop("chosen").tokens()

        for _ in range(6):
            one_step()
        settle()
        dt = _timed(torch, lambda: ([one_step() for _ in range(steps)], settle())) / steps
        ctx = engine.length(keys[0]) - steps / 2.0
        for k in keys:
            engine.end_request(k)
        got = decode_bytes(raw, batch, ctx) / dt / 1e9
        print(json.dumps(dict(base, metric=f"decode tok/s at batch {batch}, {context}-token context (Qwen3-4B shape)",
                              value=round(batch / dt, 1), unit="tok/s", ms_per_step=round(dt * 1e3, 4), steps=steps,
                              roofline={"bound": "hbm", "achieved": round(got, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                        "frac": round(got / PEAK_HBM_GBS, 4)})), flush=True)

    def prefill_point(tokens):
        def once(tag):
            engine.add_request(tag)
            toks = rand(tokens)
            dt = _timed(torch, lambda: ops.argmax_rows(engine.step([StepEntry(tag, toks, [tokens - 1])])))
            engine.end_request(tag)
            return dt

        once(("w", tokens, 0)), once(("w", tokens, 1))
        dt = min(once(("p", tokens, i)) for i in range(3))
        print(json.dumps(dict(base, metric=f"prefill tok/s at {tokens} tokens (Qwen3-4B shape)", value=round(tokens / dt, 1),
                              unit="tok/s", ms=round(dt * 1e3, 3),
                              frac=round(prefill_flops(raw, tokens) / dt / PEAK_FLOPS["bf16"], 4))), flush=True)

    def mixed_point(decoders, context, portion, prompt):
        keys = [("m", i) for i in range(decoders)]
        state = {"last": fill(keys, context)}

        def one_prompt(tag):
            engine.add_request(tag)
            toks = rand(prompt)
            for a in range(0, prompt, portion):
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
                entries.append(StepEntry(tag, toks[a:a + portion], [portion - 1] if a + portion == prompt else []))
                state["last"] = ops.argmax_rows(engine.step(entries)).tolist()[:decoders]
            engine.end_request(tag)

        one_prompt(("mw", 0)), one_prompt(("mw", 1))
        reps, per = 4, prompt // portion
        dt = _timed(torch, lambda: [one_prompt(("mp", i)) for i in range(reps)]) / (reps * per)
        for k in keys:
            engine.end_request(k)
        flops = 2.0 * (decoders + portion) * (raw["num_hidden_layers"] * layer_params(raw) ) + 2.0 * raw["vocab_size"] * raw["hidden_size"] * (decoders + 1)
        print(json.dumps(dict(base, metric=f"mixed step: {decoders} decoding requests at {context} tokens + a {portion}-token "
                                           f"prompt portion (Qwen3-4B shape)", value=round((decoders + portion) / dt, 1),
                              unit="tok/s", ms_per_step=round(dt * 1e3, 4), decode_tok_s=round(decoders / dt, 1),
                              prefill_tok_s=round(portion / dt, 1), frac_of_matrix_peak=round(flops / dt / PEAK_FLOPS["bf16"], 4),
                              frac_of_hbm_peak=round(decode_bytes(raw, decoders, context + 64) / dt / 1e9 / PEAK_HBM_GBS, 4))),
              flush=True)

    for batch in (16, 32):
        decode_point(batch, 2048, args.steps)
    decode_point(128, 1024, args.steps)
    decode_point(256, 1024, args.steps)
    for context in (8192, 16384, 32768):
        decode_point(8, context, args.steps)
    decode_point(64, 16384, min(args.steps, 16))
    prefill_point(32768)
    prefill_point(16384)
    prefill_point(8192)
    prefill_point(512)
    prefill_point(128)
    mixed_point(8, 2048, 504, 2016)      # the first four portions of a long prompt as the scheduler cuts it beside 8 decoding requests: 512 rows a step
    return 0


# ---- the Gufasun design beside Qwen3 at equal sizes -------------------------------------------------------
# Shapes that resemble a real model's layers: the widths, head counts and feed-forward size of Qwen3-4B / 8B, layers
# alternating between the matrix memory and the windowed attention, the last attention layer reading the pages of the
# one before it.  Random weights; the vocabulary is Qwen3's.
GUFASUN_SHAPES = {"4b": (QWEN3_4B, 20, 1024), "8b": (QWEN3_8B, 32, 2048)}      # (widths, mLSTM heads, window)


def gufasun_config(shape: str, layers: int) -> dict:
    q, mheads, window = GUFASUN_SHAPES[shape]
    attn = {"heads": q["num_attention_heads"], "kv_heads": q["num_key_value_heads"], "dim": q["head_dim"],
            "vdim": q["head_dim"], "scale": q["head_dim"] ** -0.5, "softcap": 30.0, "conv": 4, "mask": {"size": window},
            "q_temp": {"coef": 0.25, "every": 128}}
    mem = {"heads": mheads, "dim": q["head_dim"], "vdim": q["head_dim"], "gate_cap": 15.0}
    mlp = {"kind": "dense", "ff": q["intermediate_size"]}
    out, owner = [], None
    for i in range(layers):
        if i % 2 == 0:
            out.append({"type": "mlstm", "mixer": dict(mem), "mlp": dict(mlp)})
        else:
            mixer = dict(attn)
            if owner is not None and i >= layers - 2:
                mixer["kv_from"] = owner
            else:
                owner = i
            out.append({"type": "attention", "mixer": mixer, "mlp": dict(mlp)})
    return {"architecture": "Gufasun", "vocab": q["vocab_size"], "width": q["hidden_size"], "norm": {"eps": 1e-6},
            "embedding": {"scale": 32.0}, "canon": {"taps": 4}, "layers": out}


def _kernel_family(name: str) -> str:
    base = name.split("<")[0].split("(")[0].replace("void ", "").replace("arle::", "").strip()
    if base.startswith("Cijk") or "gemm" in base.lower() or base.startswith("Custom_Cijk"):
        return "matrix products (library and own)"
    return base


def gufasun_work(raw: dict, q: dict, tokens: int, batch: int, context: int) -> dict:
    """Ideal work of the kernels that are new with this design, per step: kernel family -> (bytes, flops) for a step of
    `tokens` rows, of which `batch` requests (decode: tokens == batch, each with `context` tokens behind it)."""
    W = raw["width"]
    a = next(l["mixer"] for l in raw["layers"] if l["type"] == "attention")
    m = next(l["mixer"] for l in raw["layers"] if l["type"] == "mlstm")
    n_att = sum(l["type"] == "attention" for l in raw["layers"])
    n_own = sum(l["type"] == "attention" and "kv_from" not in l["mixer"] for l in raw["layers"])
    n_mem = len(raw["layers"]) - n_att
    L = len(raw["layers"])
    F = raw["layers"][0]["mlp"]["ff"]
    Q, KV = a["heads"] * a["dim"], a["kv_heads"] * a["dim"]
    decode = tokens == batch
    keys = min(a["mask"]["size"], context) if decode else min(a["mask"]["size"], tokens / 2)
    S = m["heads"] * m["dim"] * m["vdim"]
    return {
        "add_layernorm": ((L + 1) * tokens * W * (4 + 4 + 4 + 4 + 2 + 2), 0),
        "causal_conv": (tokens * 2 * 2 * (L * W + n_own * (Q + 2 * KV) + (n_att - n_own) * Q), 0),
        "polynorm": (L * tokens * F * 4, 0),
        "qkv_norm_store_kernel": (tokens * 2 * 2 * (n_own * (Q + 2 * KV) + (n_att - n_own) * Q), 0),
        "attn_softcap_mfma_kernel": (n_att * batch * 2 * KV * 2 * keys if decode else 0,
                                     n_att * tokens * keys * a["heads"] * 2 * (a["dim"] + a["vdim"])),
        "mlstm_memory_kernel": (n_mem * batch * S * 4 * 2, n_mem * tokens * S * 4),
        "mlstm_gates_kernel": (n_mem * tokens * m["heads"] * m["dim"] * 2 * 2, 0),
        "mlstm_output_kernel": (n_mem * tokens * m["heads"] * m["vdim"] * (4 + 2 + 2), 0),
    }


def qwen3_work(q: dict, layers: int, tokens: int, batch: int, context: int) -> dict:
    """The like kernels of the Qwen3 model of the same widths."""
    W, F = q["hidden_size"], q["intermediate_size"]
    Q, KV, D = q["num_attention_heads"] * q["head_dim"], q["num_key_value_heads"] * q["head_dim"], q["head_dim"]
    decode = tokens == batch
    keys = context if decode else tokens / 2
    attn = (layers * batch * 2 * KV * 2 * keys if decode else 0, layers * tokens * keys * q["num_attention_heads"] * 4 * D)
    return {"rmsnorm_vec_kernel": ((layers + 1) * tokens * W * (4 + 4 + 4 + 2), 0),
            "add_stack_rmsnorm_kernel": (layers * tokens * W * (4 + 4 + 4 + 2), 0),
            "silu_mul_bf16x8_kernel": (layers * tokens * F * 6, 0),
            "qk_prep": (layers * tokens * (Q + 2 * KV) * 4, 0),
            "attn_mfma_kernel": attn, "attn_prefill_dma_kernel": attn, "attn_prefill_lds_kernel": attn}


# ---- the Sovutar design beside Qwen3 at equal sizes -------------------------------------------------------
# The widths and head counts of Qwen3-4B / 8B; layers alternate between the chunked attention (values mixed with the
# first layer's) and the latent attention (a latent of 192 and a rotated part of 64: keys of 256, the widest the
# matrix-core attention takes); sixteen experts of which four are chosen, and a shared one.
SOVUTAR_SHAPES = {"4b": (QWEN3_4B, 1024, 1536), "8b": (QWEN3_8B, 2048, 2048)}      # (widths, window and chunk, expert size)


def sovutar_config(shape: str, layers: int) -> dict:
    q, span, ff = SOVUTAR_SHAPES[shape]
    H, D = q["num_attention_heads"], q["head_dim"]
    attn = {"heads": H, "kv_heads": q["num_key_value_heads"], "dim": D, "vdim": D, "scale": D ** -0.5,
            "mask": {"size": span}, "v_mix": True}
    lat = {"heads": H, "dim": D, "rot_dim": 64, "vdim": D, "kv_rank": 192, "scale": (D + 64) ** -0.5,
           "mask": {"size": span}, "rot": {"base": 1000000.0, "dims": 64}}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": 16, "top": 4, "scale": 2.5}, "shared": {"ff": ff}}
    out = [{"type": "attention", "mixer": dict(attn), "mlp": dict(mlp)} if i % 2 == 0 else
           {"type": "latent_attention", "mixer": dict(lat), "mlp": dict(mlp)} for i in range(layers)]
    return {"architecture": "Sovutar", "vocab": q["vocab_size"], "width": q["hidden_size"], "norm": {"eps": 1e-6},
            "logit_softcap": 30.0, "layers": out}


def sovutar_work(raw: dict, q: dict, tokens: int, batch: int, context: int) -> dict:
    """Ideal work of the kernels that are new with this design, per step: kernel family -> (bytes, flops)."""
    W, L = raw["width"], len(raw["layers"])
    a = next(l["mixer"] for l in raw["layers"] if l["type"] == "attention")
    m = next(l["mixer"] for l in raw["layers"] if l["type"] == "latent_attention")
    n_att = sum(l["type"] == "attention" for l in raw["layers"])
    n_lat = L - n_att
    mlp = raw["layers"][0]["mlp"]
    E, top, F = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
    H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
    LH, LD, R, LDv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    decode = tokens == batch
    span = a["mask"]["size"]
    keys_a = (context % span if decode else min(span, tokens) / 2) or 1
    keys_l = min(m["mask"]["size"], context) if decode else min(m["mask"]["size"], tokens / 2)
    attn_bytes = (n_att * batch * keys_a * G * (D + Dv) * 2 + n_lat * batch * keys_l * (2 * C + R) * 2) if decode else 0
    attn_flops = n_att * tokens * keys_a * H * 2 * (D + Dv) + n_lat * tokens * keys_l * LH * 2 * (2 * C + R)
    active = min(E, batch * top) if decode else E
    return {
        "norm_add_kernel": (tokens * W * (L * (4 + 8 + 2) + L * ((top + 1) * 4 + 8 + 2)), 0),
        "wide_norm_store_kernel": (n_att * tokens * (H * D + G * D + G * Dv) * 4, 0),
        "latent_prep_kernel": (n_lat * tokens * (LH * R * 2 + (C + R) + 2 * C + R) * 2, 0),
        "head_proj": (n_lat * (tokens * LH * (LD + 2 * C + LDv) * 2 + LH * C * (LD + LDv) * 2),
                      n_lat * tokens * LH * C * (LD + LDv) * 2),
        "attn_softcap_mfma_kernel": (attn_bytes, attn_flops),
        "moe_route_kernel": (L * (tokens + E) * W * 2, 0),
        "moe_expert": (L * (active * 3 * W * F * 2 + tokens * top * (W * 2 + F * 4 + W * 4)), L * tokens * top * 3 * W * F * 2),
    }


# ---- the Tazitar design beside Qwen3 at equal sizes -------------------------------------------------------
# The widths and head counts of Qwen3-4B / 8B over four residual streams; the layers cycle through the three mixers
# (capped attention with q/k norm; an attention with a sink beside a gated delta rule; an attention with interleaved
# YaRN rotation and a learned sink), and from eight layer runs on, layers 1..3 run twice with the same weights.
def tazitar_config(shape: str, layers: int) -> dict:
    q = SOVUTAR_SHAPES[shape][0]
    H, G, D = q["num_attention_heads"], q["num_key_value_heads"], q["head_dim"]
    attn = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "softcap": 30.0,
            "rot": {"base": 1000000.0, "dims": D}}
    left = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": 0.3, "rot": {"base": 1000000.0, "dims": D // 2}}
    right = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "conv": 4}
    attn2 = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": 0.3,
             "rot": {"base": 1000000.0, "dims": D, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
    kinds = [("attention", attn), ("parallel", {"left": left, "right": right}), ("attention_2", attn2)]
    mlp = {"kind": "dense", "ff": q["intermediate_size"]}
    loop = {"start": 1, "stop": 4, "times": 2} if layers >= 8 else None
    unique = layers - 3 if loop else layers
    out = [{"type": kinds[i % 3][0], "mixer": json.loads(json.dumps(kinds[i % 3][1])), "mlp": dict(mlp)} for i in range(unique)]
    raw = {"architecture": "Tazitar", "vocab": q["vocab_size"], "width": q["hidden_size"], "norm": {"eps": 1e-6},
           "streams": 4, "layers": out}
    if loop:
        raw["loop"] = loop
    return raw


def tazitar_work(raw: dict, q: dict, tokens: int, batch: int, context: int) -> dict:
    """Ideal work of the kernels that are new with this design, per step: kernel family -> (bytes, flops)."""
    from arle_amd.config import TazitarConfig

    order = TazitarConfig.from_dict(raw).layer_order()
    runs = [raw["layers"][i] for i in order]
    W, S, L = raw["width"], raw["streams"], len(runs)
    F = runs[0]["mlp"]["ff"]
    n_par = sum(l["type"] == "parallel" for l in runs)
    a = next(l["mixer"] for l in runs if l["type"] == "attention")
    r = next(l["mixer"]["right"] for l in runs if l["type"] == "parallel") if n_par else None
    H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
    decode = tokens == batch
    keys = context if decode else tokens / 2
    work = {
        "hyper_step_kernel": ((2 * L + 1) * tokens * W * (8 * S + 4 + 2), 0),
        "rotary_qkv_store_x8_kernel": (L * tokens * (H * D + G * D + G * Dv) * 4, 0),
        "attn_softcap_mfma_kernel": (L * batch * keys * G * (D + Dv) * 2 if decode else 0, L * tokens * keys * H * 2 * (D + Dv)),
        "silu_mul_bf16x8_kernel": (L * tokens * F * 6, 0),
    }
    if r is not None:
        state = r["heads"] * r["dim"] * r["vdim"]
        conv = 2 * r["kv_heads"] * r["dim"] + r["heads"] * r["vdim"]
        work.update({
            "pair_norm_kernel": (n_par * tokens * W * 12, 0),
            "causal_conv": (n_par * tokens * conv * 4, 0),
            "gated_delta_scan_kernel": (n_par * batch * state * 8, n_par * tokens * state * 6),
            "gated_delta_output_kernel": (n_par * tokens * r["heads"] * r["vdim"] * 8, 0),
        })
    return work


# ---- the Retudra design beside Sovutar and Qwen3 at equal sizes ------------------------------------------
# The widths and head counts of Qwen3-4B / 8B; the layers cycle through the windowed attention that keeps its first
# keys, the delta rule with a decay a key channel and the gated latent attention (Sovutar's sizes: a latent of 192 and a
# rotated part of 64); the first layer's feed-forward is dense, the others have sixteen experts and two identity experts
# in three groups of which two are kept, four choices a token; a token-side input of 256 columns a layer.
def retudra_config(shape: str, layers: int) -> dict:
    q, span, ff = SOVUTAR_SHAPES[shape]
    H, G, D = q["num_attention_heads"], q["num_key_value_heads"], q["head_dim"]
    attn = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "rot": {"base": 1000000.0, "dims": D // 2},
            "mask": {"size": span, "keep_first": 64}}
    lat = {"heads": H, "dim": D, "rot_dim": 64, "vdim": D, "kv_rank": 192, "scale": (D + 64) ** -0.5,
           "rot": {"base": 1000000.0, "dims": 64}}
    dlt = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "conv": 4, "decay_rank": 64, "gate_rank": 64}
    kinds = [("attention", attn), ("channel_delta", dlt), ("latent_attention", lat)]
    moe = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": 16, "top": 4, "identity": 2, "groups": {"count": 3, "keep": 2}}}
    out = [{"type": kinds[i % 3][0], "mixer": json.loads(json.dumps(kinds[i % 3][1])),
            "mlp": {"kind": "dense", "ff": q["intermediate_size"]} if i == 0 else json.loads(json.dumps(moe))}
           for i in range(layers)]
    return {"architecture": "Retudra", "vocab": q["vocab_size"], "width": q["hidden_size"], "norm": {"eps": 1e-6},
            "residual_mult": 0.5, "token_side": {"dim": 256}, "logit_softcap": 30.0, "layers": out}


def retudra_work(raw: dict, q: dict, tokens: int, batch: int, context: int) -> dict:
    """Ideal work of the design's kernels, per step: kernel family -> (bytes, flops)."""
    W, L = raw["width"], len(raw["layers"])
    of = lambda kind: [l for l in raw["layers"] if l["type"] == kind]
    n_att, n_dlt, n_lat = len(of("attention")), len(of("channel_delta")), len(of("latent_attention"))
    moes = [l["mlp"] for l in raw["layers"] if l["mlp"] and l["mlp"]["kind"] == "moe"]
    decode = tokens == batch
    work = {"token_gate_kernel": (L * tokens * raw["token_side"]["dim"] * 6, 0)}
    top = moes[0]["router"]["top"] if moes else 0
    # a norm on a sublayer's output: the addend (32-bit; the experts' `top` outputs), the residual in and out, its rounded copy
    work["norm_add_kernel"] = (tokens * W * ((2 * L + (L - len(moes))) * 14 + len(moes) * (top * 4 + 10)), 0)
    if n_att:
        a = of("attention")[0]["mixer"]
        H, G, D, Dv, span = a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["mask"]["size"]
        keys = min(span + a["mask"]["keep_first"], context) if decode else min(span, tokens / 2)
        work["wide_norm_store_kernel"] = (n_att * tokens * (H * D + G * D + G * Dv) * 4, 0)
        att_bytes = n_att * batch * keys * G * (D + Dv) * 2 if decode else 0
        att_flops = n_att * tokens * keys * H * 2 * (D + Dv)
    else:
        att_bytes = att_flops = 0
    if n_lat:
        m = of("latent_attention")[0]["mixer"]
        LH, LD, R, LDv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        keys = context if decode else tokens / 2
        att_bytes += n_lat * batch * keys * (2 * C + R) * 2 if decode else 0
        att_flops += n_lat * tokens * keys * LH * 2 * (2 * C + R)
        work["latent_prep_kernel"] = (n_lat * tokens * (LH * R * 2 + (C + R) + 2 * C + R) * 2, 0)
        work["head_proj"] = (n_lat * (tokens * LH * (LD + 2 * C + LDv) * 2 + LH * C * (LD + LDv) * 2),
                             n_lat * tokens * LH * C * (LD + LDv) * 2)
        work["gate_mul"] = (n_lat * tokens * LH * LDv * 6, 0)
    work["attn_softcap_mfma_kernel"] = (att_bytes, att_flops)
    if n_dlt:
        r = of("channel_delta")[0]["mixer"]
        state = r["heads"] * r["dim"] * r["vdim"]
        conv = 2 * r["kv_heads"] * r["dim"] + r["heads"] * r["vdim"]
        work.update({"causal_conv": (n_dlt * tokens * conv * 4, 0),
                     "gated_delta_scan_kernel": (n_dlt * (batch * state * 8 + tokens * r["heads"] * r["dim"] * 4), n_dlt * tokens * state * 8),
                     "gated_delta_output_kernel": (n_dlt * tokens * r["heads"] * r["vdim"] * 8, 0)})
    if moes:
        E, F = moes[0]["router"]["experts"], moes[0]["expert"]["ff"]
        outputs = E + moes[0]["router"].get("identity", 0)
        active = min(E, batch * top) if decode else E
        n = len(moes)
        work.update({"moe_route_kernel": (n * (tokens + outputs) * W * 2, 0),
                     "moe_expert": (n * (active * 3 * W * F * 2 + tokens * top * (W * 2 + F * 4 + W * 4)), n * tokens * top * 3 * W * F * 2),
                     "moe_identity_kernel": (n * tokens * top * W * 6 * moes[0]["router"].get("identity", 0) / outputs, 0)})
    return work


def retudra_bench(args) -> int:
    """Prefill and decode throughput of the Retudra design, of Sovutar (the closest design: sublayers normed on their
    way out, a latent attention, a mixture of experts) and of Qwen3 at the same widths and depth."""
    from arle_amd.config import Qwen3Config, RetudraConfig, SovutarConfig

    layers = args.layers if args.layers != FULL_LAYERS else 8
    q = dict(SOVUTAR_SHAPES[args.shape][0], num_hidden_layers=layers)
    raw, sov = retudra_config(args.shape, layers), sovutar_config(args.shape, layers)
    models = {"retudra": ("Retudra", RetudraConfig.from_dict(raw)), "sovutar": ("Sovutar", SovutarConfig.from_dict(sov)),
              "qwen3": ("Qwen3ForCausalLM", Qwen3Config.from_dict(q))}
    return design_bench(args, "retudra", models, q, layers, lambda tokens, batch, context: retudra_work(raw, q, tokens, batch, context),
                        {"sovutar": lambda tokens, batch, context: sovutar_work(sov, q, tokens, batch, context)})


def tazitar_bench(args) -> int:
    """Prefill and decode throughput of the Tazitar design and of Qwen3 at the same widths and depth."""
    from arle_amd.config import Qwen3Config, TazitarConfig

    layers = args.layers if args.layers != FULL_LAYERS else 8
    q = dict(SOVUTAR_SHAPES[args.shape][0], num_hidden_layers=layers)
    raw = tazitar_config(args.shape, layers)
    models = {"tazitar": ("Tazitar", TazitarConfig.from_dict(raw)), "qwen3": ("Qwen3ForCausalLM", Qwen3Config.from_dict(q))}
    return design_bench(args, "tazitar", models, q, layers, lambda tokens, batch, context: tazitar_work(raw, q, tokens, batch, context))


def sovutar_bench(args) -> int:
    """Prefill and decode throughput of the Sovutar design and of Qwen3 at the same widths and depth."""
    from arle_amd.config import Qwen3Config, SovutarConfig

    layers = args.layers if args.layers != FULL_LAYERS else 8
    q = dict(SOVUTAR_SHAPES[args.shape][0], num_hidden_layers=layers)
    raw = sovutar_config(args.shape, layers)
    models = {"sovutar": ("Sovutar", SovutarConfig.from_dict(raw)), "qwen3": ("Qwen3ForCausalLM", Qwen3Config.from_dict(q))}
    return design_bench(args, "sovutar", models, q, layers, lambda tokens, batch, context: sovutar_work(raw, q, tokens, batch, context))


def gufasun_bench(args) -> int:
    """Prefill and decode throughput of the Gufasun design and of Qwen3 at the same widths and depth."""
    from arle_amd.config import GufasunConfig, Qwen3Config

    layers = args.layers if args.layers != FULL_LAYERS else 8
    q = dict(GUFASUN_SHAPES[args.shape][0], num_hidden_layers=layers)
    raw = gufasun_config(args.shape, layers)
    models = {"gufasun": ("Gufasun", GufasunConfig.from_dict(raw)), "qwen3": ("Qwen3ForCausalLM", Qwen3Config.from_dict(q))}
    return design_bench(args, "gufasun", models, q, layers, lambda tokens, batch, context: gufasun_work(raw, q, tokens, batch, context))


def design_bench(args, design: str, models: dict, q: dict, layers: int, design_work, other_work: dict | None = None) -> int:
    """Prefill and decode throughput of a design and of Qwen3 (and further models) at the same widths and depth, one JSON
    line each, and the time of a step by kernel family with what each new kernel reaches of its roofline.
    other_work: {model name: its ideal work} for models beside the design and Qwen3."""
    import torch

    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops

    batch, prompt = args.batch or 8, args.prompt_len
    gen = torch.Generator().manual_seed(1234)
    toks = lambda n: torch.randint(0, q["vocab_size"], (n,), generator=gen).tolist()
    lines = []
    for name, (arch, config) in models.items():
        engine = Engine.from_config(arch, config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                    max_tokens=(batch + 1) * (prompt + 256), max_slots=batch + 1,
                                    max_request_tokens=prompt + 256)

        def prefill_once(key):
            engine.add_request(key)
            t = toks(prompt)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ops.argmax_rows(engine.step([StepEntry(key, t, [prompt - 1])]))
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            engine.end_request(key)
            return dt

        for i in range(3):
            prefill_once(("warm", i))
        prefill_s = min(prefill_once(("p", i)) for i in range(5))
        keys = [("d", i) for i in range(batch)]
        last = []
        for k in keys:
            engine.add_request(k)
            last += ops.argmax_rows(engine.step([StepEntry(k, toks(prompt), [prompt - 1])])).tolist()

        def decode_step():
            nonlocal last
            last = ops.argmax_rows(engine.step([StepEntry(k, [t], [0]) for k, t in zip(keys, last)])).tolist()

        for _ in range(args.warmup):
            decode_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            decode_step()
        torch.cuda.synchronize()
        decode_s = (time.perf_counter() - t0) / args.steps
        line = {"metric": f"{name} at the Qwen3-{args.shape.upper()} widths, {layers} layers, random weights", "dtype": "bf16",
                "prefill_tok_s": round(prompt / prefill_s, 1), "prefill_ms": round(prefill_s * 1e3, 3), "prompt": prompt,
                "decode_tok_s": round(batch / decode_s, 1), "decode_ms": round(decode_s * 1e3, 3), "batch": batch}
        if not args.no_parts:
            engine.use_graphs = False        # the profiler names the kernels of eager steps
            engine.add_request("prof")
            t = toks(prompt)
            pre, dec = profiled_steps(torch, [lambda: engine.step([StepEntry("prof", t, [prompt - 1])]), decode_step])
            engine.end_request("prof")
            ideal = design_work if name == design else (other_work or {}).get(
                name, lambda tokens, rows, context: qwen3_work(q, layers, tokens, rows, context))
            work = {"prefill": ideal(prompt, 1, 0), "decode": ideal(batch, batch, prompt)}
            for phase, step in (("prefill", pre), ("decode", dec)):
                fam: dict = {}
                for kname, us in step:
                    f = fam.setdefault(_kernel_family(kname), [0, 0.0])
                    f[0] += 1
                    f[1] += us
                table = {}
                for f, (count, us) in sorted(fam.items(), key=lambda kv: -kv[1][1]):
                    row = {"launches": count, "us": round(us, 1)}
                    match = next((w for key, w in work[phase].items() if f.startswith(key)), None)
                    if match is not None and us > 0:
                        row["of_roofline"] = round(max(match[0] / (PEAK_HBM_GBS * 1e9), match[1] / PEAK_FLOPS["bf16"]) / (us * 1e-6), 4)
                    table[f] = row
                line[phase + "_kernels"] = table
        print(json.dumps(line), flush=True)
        lines.append(line)
        for k in keys:
            engine.end_request(k)
        del engine
        torch.cuda.empty_cache()
    return 0


def main() -> int:
    global PAGE, PROMPT
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=None, help="decoding requests (default: 8; 64 for qwen3-32b-decode)")
    ap.add_argument("--context", type=int, default=8192, help="tokens of context of the qwen3-32b-decode workload")
    ap.add_argument("--layers", type=int, default=FULL_LAYERS)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-size", type=int, default=PAGE, help="tokens per cache page")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 decode points")
    ap.add_argument("--no-overlap", action="store_true",
                    help="decode steps wait for their tokens on the host before the next is prepared (default: the "
                         "next step is launched from the tokens on the GPU, as the scheduler does)")
    ap.add_argument("--no-weight-tiles", action="store_true",
                    help="without the second copy of the projection weights that the few-rows kernels stream")
    ap.add_argument("--no-parts", action="store_true",
                    help="skip the breakdown of the step's time by part of the model (a profiled step)")
    ap.add_argument("--parts-only", action="store_true",
                    help="print only that breakdown (what the default run starts as a child process, after its own timing)")
    ap.add_argument("--ceilings", action="store_true",
                    help="measure what a kernel that only reads, and one that only multiplies, reach on this GPU, and exit")
    ap.add_argument("--prompt-len", type=int, default=PROMPT,
                    help="tokens of the prefill that --prefill-only measures and of the prompts of --generate (default 2,048)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="measure the 2,048-token prefill alone (for profiles of its kernels) and print that")
    ap.add_argument("--gaps", action="store_true",
                    help="decode steps that wait for their tokens against steps launched ahead: time a step, GPU busy and idle")
    ap.add_argument("--first-token", action="store_true",
                    help="time to the first token through LLM.generate, portions by the GPU's memory against portions of 512")
    ap.add_argument("--generate", action="store_true",
                    help="the decode workload as a user runs it: 1, 8 and 64 prompts of --prompt-len tokens, 256 generated each, "
                         "through LLM.generate")
    ap.add_argument("--sweep", action="store_true",
                    help="further sizes of the Qwen3-4B shape (batch 16/32, 8k/32k context, 8,192-token prefill, portions "
                         "beside decoding requests), one JSON line each")
    ap.add_argument("--tune-products", metavar="WIDTHS", default=None,
                    help="time every kernel that can run each of a layer's four matrix products, row count by row count, "
                         "and write the table that ARLE_AMD_PRODUCT_TABLE / ops.load_product_table reads; WIDTHS: 4b, 8b, "
                         "32b or hidden,q_width,kv_width,intermediate[,vocabulary]")
    ap.add_argument("--out", default=None, help="--tune-products: the table's file (default: product_table_<widths>.json)")
    ap.add_argument("--workload", default="qwen3-4b", choices=["qwen3-4b", "qwen3-8b-mixed", "qwen3-32b-decode", "gufasun", "sovutar", "tazitar", "retudra"],
                    help="qwen3-4b is the default run; the next two are further workloads at larger shapes; gufasun: "
                         "the Gufasun design beside Qwen3 at equal widths and depth (--shape, --layers, --batch, --prompt-len)")
    ap.add_argument("--shape", default="4b", choices=["4b", "8b"], help="--workload gufasun / sovutar / tazitar / retudra: whose widths")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for --gpus {args.gpus})")
        return 2
    PAGE = args.page_size
    if args.prefill_only:
        PROMPT = args.prompt_len
    if args.ceilings:
        return ceilings()
    if args.tune_products:
        return tune_products(args)
    if args.sweep:
        return sweep(args)
    if args.first_token:
        return first_token(args)
    if args.generate:
        return generate_workload(args)
    if args.gaps:
        return step_gaps(args)
    if args.workload == "gufasun":
        return gufasun_bench(args)
    if args.workload == "sovutar":
        return sovutar_bench(args)
    if args.workload == "tazitar":
        return tazitar_bench(args)
    if args.workload == "retudra":
        return retudra_bench(args)
    if args.workload == "qwen3-4b" and args.batch is None:
        args.batch = 8
    if args.workload != "qwen3-4b":
        if args.layers == FULL_LAYERS:
            args.layers = 0   # the workload's own depth
        return mixed_8b(args) if args.workload == "qwen3-8b-mixed" else decode_32b(args)

    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops
    from arle_amd.sampling import Sampler, SamplingParams

    raw = dict(QWEN3_4B, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    elt = 2 if dkey == "bf16" else 4
    max_batch = args.batch if (args.no_points or args.parts_only or args.prefill_only) else max(args.batch, 64)
    longest = max(CONTEXT, PROMPT + 64)    # --prompt-len may ask for a longer prefill than the default run's context
    t0 = time.time()
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype=args.dtype,
                                page_size=PAGE, max_tokens=(max_batch + 1) * longest, max_slots=max_batch + 1,
                                max_request_tokens=longest, weight_tiles=False if args.no_weight_tiles else None)
    print(f"[bench] engine ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(1234)
    sampler = Sampler(engine.device)       # the product's sampler: greedy rows are one argmax kernel, read back on its own stream
    greedy_rows = [(SamplingParams(), 0, 0, [])] * (max_batch + 1)

    def prompt_tokens(n):
        return torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()

    def timed(fn):
        torch.cuda.synchronize()
        t = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t

    # ---- prefill: one 2,048-token prompt, logits of its last token included -----------------
    def prefill_once(key):
        engine.add_request(key)
        toks = prompt_tokens(PROMPT)
        dt = timed(lambda: ops.argmax_rows(engine.step([StepEntry(key, toks, [PROMPT - 1])])))
        engine.end_request(key)
        return dt


    for i in range(5):      # eager, captured, then replays until the clocks have settled (the sixth run is as fast as the twentieth)
        prefill_once(("warm", i))
    prefill_s = min(prefill_once(("prefill", i)) for i in range(5))
    prefill = {"value": round(PROMPT / prefill_s, 1), "tokens": PROMPT, "ms": round(prefill_s * 1e3, 3),
               "frac": round(prefill_flops(raw, PROMPT) / prefill_s / PEAK_FLOPS[dkey], 4)}
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    if args.prefill_only:
        print(json.dumps({"metric": f"prefill tok/s at {PROMPT} tokens (Qwen3-4B shape, random weights)",
                          "value": prefill["value"], "unit": "tok/s", "n_gpus": 1, "dtype": dkey,
                          "higher_is_better": True, "prefill": prefill}))
        return 0

    # ---- decode ---------------------------------------------------------------------------------
    def decode_run(batch, steps, warmup, parts=False):
        """(seconds of `steps` timed steps, mean context); with `parts` instead the breakdown of a step's time."""
        keys = [("d", batch, i) for i in range(batch)]
        last = []
        for k in keys:
            engine.add_request(k)
        per_step = max(1, 8192 // PROMPT)
        for i in range(0, batch, per_step):   # real prefill of every request, a few prompts a step
            group = keys[i:i + per_step]
            out = engine.step([StepEntry(k, prompt_tokens(PROMPT), [PROMPT - 1]) for k in group])
            last.extend(ops.argmax_rows(out).tolist())
        state = {"last": last, "chosen": None}

        def one_step():
            """A decode step as the scheduler runs it (Scheduler._run_ahead): launched from the tokens that the
            step before left on the GPU, which the host reads back while this step runs.  --no-overlap: every
            step waits for its tokens on the host before the next is prepared."""
            if args.no_overlap or parts:
                out = engine.step([StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])])
                state["last"] = ops.argmax_rows(out).tolist()   # the host needs the token to go on
                return
            before = state["chosen"]
            if before is None:
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
            else:
                entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
            state["chosen"] = sampler.choose(engine.step(entries, borrow_logits=True), greedy_rows[:batch])
            if before is not None:
                state["last"] = before.tokens()                 # the step before: every token reaches the host

        def settle():
            if state["chosen"] is not None:
                state["last"] = state["chosen"].tokens()
                state["chosen"] = None

        for _ in range(warmup):
            one_step()
        ctx0 = engine.length(keys[0])
        settle()
        dt = timed(lambda: ([one_step() for _ in range(steps)], settle()))   # the last step's tokens are read inside
        ctx_mean = ctx0 + (steps - 1) / 2.0 + 1
        if parts:
            from arle_amd.kernels import ceilings as measured

            read_ceiling = measured.read_bandwidth(total_bytes=1 << 30, repeats=3)["best"]
            mfma_ceiling = max(measured.mfma_rate(shape=32, iters=4000, repeats=2),
                               measured.mfma_rate(shape=16, iters=4000, repeats=2))
            ctx_now = engine.length(keys[0]) + 2
            calls = [lambda: prefill_once(("parts", 0))] * 3 + [one_step] * 5
            traced = profiled_steps(torch, calls)
            out = {"ceilings": {"hbm_read_gbs": round(read_ceiling / 1e9, 1), "mfma_tflops": round(mfma_ceiling / 1e12, 1)}}
            times = part_times(traced[:3], args.layers)
            flops = part_flops_prefill(raw, PROMPT)
            head_flops = flops.pop("head")      # one row against the whole table: a stream of weights, judged by its bytes
            us, of_peak, of_ceiling = part_report(times, flops, PEAK_FLOPS[dkey], mfma_ceiling)
            head_bytes = raw["vocab_size"] * raw["hidden_size"] * elt
            of_peak["head_hbm"] = round(head_bytes / (times["head"] * 1e-6) / (PEAK_HBM_GBS * 1e9), 4)
            of_ceiling["head_hbm"] = round(head_bytes / (times["head"] * 1e-6) / read_ceiling, 4)
            # the profiled pass is longer than the timed one (the profiler's own cost a kernel): both are given
            us["sum"] = round(sum(v for k, v in us.items() if k != "kernels"), 1)
            out.update(prefill_parts_us=us, prefill_parts_frac_peak=of_peak, prefill_parts_frac_ceiling=of_ceiling)
            us, of_peak, of_ceiling = part_report(part_times(traced[3:], args.layers),
                                                  part_bytes_decode(raw, batch, ctx_now, elt), PEAK_HBM_GBS * 1e9, read_ceiling)
            us["sum"] = round(sum(v for k, v in us.items() if k != "kernels"), 1)
            out.update(decode_parts_us=us, decode_parts_frac_peak=of_peak, decode_parts_frac_ceiling=of_ceiling)
            for k in keys:
                engine.end_request(k)
            return out
        for k in keys:
            engine.end_request(k)
        return dt, ctx_mean

    if args.parts_only:
        print(json.dumps(decode_run(args.batch, 4, 6, parts=True)))
        return 0
    dt, ctx_mean = decode_run(args.batch, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    achieved = decode_bytes(raw, args.batch, ctx_mean, elt) / (dt / args.steps) / 1e9
    print(f"[bench] decode b{args.batch}: {value:.1f} tok/s, {ms_per_step:.3f} ms/step", file=sys.stderr, flush=True)
    points = {}
    if not args.no_points:
        for b in (1, 64):
            steps = min(args.steps, 32) if b == 64 else args.steps
            d, _ = decode_run(b, steps, max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(b * steps / d, 1)
            print(f"[bench] decode b{b}: {points[f'decode_b{b}']} tok/s", file=sys.stderr, flush=True)

    line = {
        "metric": "decode tok/s at batch 8, 2,048-token prompts (Qwen3-4B shape, random weights)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey, "data": "synthetic: seeded random weights N(0,0.02), uniform random token ids",
        "config": {"model": "Qwen3-4B shape", "global_batch": args.batch, "seq_len": CONTEXT, "prompt_len": PROMPT,
                   "parallelism": "single GPU", "layers": args.layers, "layers_full": FULL_LAYERS,
                   "hidden": raw["hidden_size"], "q_heads": raw["num_attention_heads"],
                   "kv_heads": raw["num_key_value_heads"], "head_dim": raw["head_dim"],
                   "intermediate": raw["intermediate_size"], "vocab": raw["vocab_size"],
                   "rope_theta": raw["rope_theta"], "rms_norm_eps": raw["rms_norm_eps"], "tied": True,
                   "page_size": PAGE, "weight_tiles": engine.rt.weight_tiles,
                   "readback_lag_steps": 0 if args.no_overlap else 1},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }
    if not args.no_parts and dkey == "bf16":
        line.update(parts_in_a_child_process(args))
        # the parts come from a second, profiled run: their sums stand beside the timed steps they are read against
        if isinstance(line.get("prefill_parts_us"), dict):
            line["prefill_parts_us"]["timed_step"] = round(prefill["ms"] * 1e3, 1)
            line["decode_parts_us"]["timed_step"] = round(ms_per_step * 1e3, 1)
    if args.batch != 8:
        line["metric"] = line["metric"].replace("batch 8", f"batch {args.batch}")
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
