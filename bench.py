"""Decode and prefill throughput of the Llama-3.2-1B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one decode step of the whole engine (scheduler, step function, kernels, sampling) at
batch 8 with 2,048-token contexts that grow while decoding. Prints ONE JSON line. The same line
carries the 2,048-token prefill, the decode step's HBM roofline, and decode at batch 1 and 64.

    python bench.py --kernel-classes [--batch B]

times the kernels of one decode step class by class (qkv, attention, o, gate|up, down, norms, head,
sampling) with events around each launch of an eager step, and prints the bytes each class has to
read, its time and its rate beside the step's total, as one JSON line.

    python bench.py --designs [--shape 1b|3b] [--layers L]

measures the Rugezen decoder (parallel layers on a 32-bit stream, attention with head norms, capped
scores and a sink, a minGRU every fourth layer, dense squared-relu feed-forward) beside the Llama
decoder at equal layer sizes and equal parameter count, random weights: prefill tokens/s and decode
tokens/s at batch 1, 8 and 64 through the whole engine, and kernel by kernel the pairs of like kernels
(attention over prompt portions and over decoded tokens, rotation and cache write, residual sum and
norms, the feed-forward's activation) with the bytes or operations each has to move and what share of
the machine's peak that comes to. One JSON line.

    python bench.py --fanotar [--shape 1b|3b] [--layers L]

measures the Fanotar decoder (dynamic-tanh norms around every part on a 32-bit stream, attention behind a
short convolution with distance slopes, learned sinks, a window and an output gate, every fourth layer
reading its neighbour's cache, capped gated feed-forward, dense and as a mixture of experts in turn) beside
the Rugezen decoder, the closest of the engine's models, at equal layer sizes and equal active parameters
per token, in the same way: whole-engine throughput and the like kernels side by side. One JSON line.

    python bench.py --bafarax [--shape 1b|3b] [--layers L] [--kernels-only]

measures the Bafarax decoder (pre-norm layers on a 32-bit stream whose mixers are, in turn, attention inside chunks
with a norm over the whole projections and learned sinks, attention through a low-rank latent with a window and an
output gate, and an mLSTM's matrix memory; dense and ungated routed feed-forwards) beside the Fanotar decoder, the
closest of the engine's models, at equal layer sizes and equal active parameters per token, in the same way. One JSON
line.

    python bench.py --tegolix [--shape 1b|3b] [--layers L] [--kernels-only]

measures the Tegolix decoder (sandwiched RMS norms and learned scales per channel on a 32-bit stream, a per-layer token
input, gated linear attention in turn with windowed attention beside a recurrence with token shift, dense and routed
feed-forwards with identity experts and a gated shared expert) beside the Bafarax decoder, the closest of the engine's
models, at equal layer sizes, in the same way. One JSON line.

    python bench.py --scenario requests-3b | chunked-8b [--layers L]

runs a whole workload through `LLM.generate` instead and prints one JSON line of its own: many
requests that arrive together, at the layer sizes of Llama 3.2 3B (prompts of 512 to 4,096 tokens, a
quarter of them behind a common 1,024-token prefix, prefix cache on) or of Llama 3.1 8B (8,192-token
contexts whose prompts are fed in portions of 2,048 tokens beside the decoding requests).
"""

from __future__ import annotations

import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# layer sizes (--shape); the default, "1b", is the one the headline numbers are quoted on
SHAPES = {
    "1b": dict(model="llama-3.2-1b-shape", layers_full=16, rope_factor=32.0,
               shape=dict(vocab_size=128256, hidden_size=2048, intermediate_size=8192, num_attention_heads=32,
                          num_key_value_heads=8, head_dim=64, max_position_embeddings=131072, rms_norm_eps=1e-5,
                          rope_theta=500000.0, tie_word_embeddings=True)),
    "3b": dict(model="llama-3.2-3b-shape", layers_full=28, rope_factor=32.0,
               shape=dict(vocab_size=128256, hidden_size=3072, intermediate_size=8192, num_attention_heads=24,
                          num_key_value_heads=8, head_dim=128, max_position_embeddings=131072, rms_norm_eps=1e-5,
                          rope_theta=500000.0, tie_word_embeddings=True)),
    "8b": dict(model="llama-3.1-8b-shape", layers_full=32, rope_factor=8.0,
               shape=dict(vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_attention_heads=32,
                          num_key_value_heads=8, head_dim=128, max_position_embeddings=131072, rms_norm_eps=1e-5,
                          rope_theta=500000.0, tie_word_embeddings=False)),
}
ROPE = dict(factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)
PROMPT_LEN, MAX_MODEL_LEN, PAGE = 2048, 4096, 256
SHAPE = SHAPES["1b"]["shape"]

# whole workloads: layer sizes, requests, and how the scheduler is set for them
SCENARIOS = {
    "requests-3b": dict(**SHAPES["3b"], requests=64, prompt=(512, 4096), shared=(0.25, 1024), decode=256, budget=8192,
                        chunk=0, caching=True),
    "chunked-8b": dict(**SHAPES["8b"], requests=32, prompt=(7936, 7936), shared=(0.0, 0), decode=256,
                       budget=2048 + 32, chunk=2048, caching=False),
}


def scenario(name: str, layers: int | None, dtype_name: str) -> int:
    """One workload from first request to last token through `LLM.generate`; one JSON line."""
    import torch

    from tinyserve_llm_amd.config import LlamaConfig, RopeScaling
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.loading import random_model
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams

    w = SCENARIOS[name]
    layers = layers or w["layers_full"]
    config = LlamaConfig(num_hidden_layers=layers, rope_scaling=RopeScaling(**{**ROPE, "factor": w["rope_factor"]}),
                         **w["shape"])
    dtype = torch.bfloat16 if dtype_name == "bf16" else torch.float32
    model = random_model(config, 0, dtype, "cuda:0")
    rng = random.Random(0)
    lo, hi = w["prompt"]
    share, prefix_len = w["shared"]
    prefix = [rng.randrange(config.vocab_size) for _ in range(prefix_len)]
    prompts = []
    for i in range(w["requests"]):
        n = rng.randint(lo, hi)
        head = prefix if i < share * w["requests"] and n > prefix_len else []
        prompts.append(head + [rng.randrange(config.vocab_size) for _ in range(n - len(head))])
    rng.shuffle(prompts)
    max_len = hi + w["decode"]
    pages = sum(-(-(len(p) + w["decode"]) // PAGE) for p in prompts) + 8
    sc = SchedulerConfig(max_model_len=max_len, max_num_seqs=w["requests"], max_num_batched_tokens=w["budget"],
                         max_prefill_chunk=w["chunk"])
    sp = SamplingParams(max_tokens=w["decode"], temperature=0.0, ignore_eos=True)

    def run(subset) -> tuple[float, LLM]:
        llm = LLM(None, sc, CacheConfig(block_size=PAGE, caching=w["caching"]), dtype=dtype, num_blocks=pages,
                  seed=0, model=model)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        llm.generate(subset, sp)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, llm

    # once untimed, with other tokens of the same lengths: libraries pick and time their kernels for
    # the batch sizes the workload meets (kept for the process); the timed run has a fresh engine
    cold_seconds, cold = run([[rng.randrange(config.vocab_size) for _ in p] for p in prompts])
    recorded_cold = cold.runner.graphs.recorded if cold.runner.graphs is not None else 0
    del cold
    seconds, llm = run(prompts)
    st, cs = llm.scheduler.stats(), llm.manager.stats()
    portions = [r for r in llm.steps if r.num_tokens > r.num_seqs]
    decodes = [r for r in llm.steps if r.num_tokens == r.num_seqs]
    prompt_tokens = sum(len(p) for p in prompts)
    record = {
        "metric": f"tokens/s of a whole workload ({name})", "value": (prompt_tokens + st.decode_tokens) / seconds,
        "unit": "tokens/s", "n_gpus": 1, "seconds": seconds, "steps": len(llm.steps), "higher_is_better": True,
        # the same workload's first run in the process: decode steps recorded as their batch sizes are first met,
        # the matrix library's candidates timed once per shape
        "cold_seconds": cold_seconds, "decode_steps_recorded_cold": recorded_cold,
        "dtype": dtype_name, "data": "synthetic uniform token ids, random weights N(0,0.02)",
        "output_tokens_per_s": st.decode_tokens / seconds, "prompt_tokens": prompt_tokens,
        "prefilled_tokens": st.prefill_tokens, "cached_tokens": st.cached_tokens, "output_tokens": st.decode_tokens,
        "preemptions": st.preemptions, "evictions": cs.evictions,
        "steps_with_prompt_portions": {"steps": len(portions), "seconds": sum(r.end - r.start for r in portions),
                                       "tokens": sum(r.num_tokens for r in portions)},
        "steps_of_decodes_only": {"steps": len(decodes), "seconds": sum(r.end - r.start for r in decodes),
                                  "tokens": sum(r.num_tokens for r in decodes)},
        "config": {"model": w["model"], "layers": layers, "layers_full": w["layers_full"],
                   "hidden": config.hidden_size, "heads": config.num_attention_heads,
                   "kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
                   "intermediate": config.intermediate_size, "vocab": config.vocab_size, "requests": w["requests"],
                   "prompt_min": lo, "prompt_max": hi, "shared_prefix": prefix_len, "decode_tokens": w["decode"],
                   "token_budget": w["budget"], "prefill_chunk": w["chunk"], "page_size": PAGE, "pages": pages},
    }
    print(json.dumps(record))
    return 0


def designs(args) -> int:
    """The Rugezen decoder beside the Llama decoder at the layer sizes of `--shape`: whole-engine
    throughput, and the like kernels of the two side by side. One JSON line."""
    import torch

    from tinyserve_llm_amd.config import LlamaConfig, RopeScaling
    from tinyserve_llm_amd.config.rugezen import RugezenAttention, RugezenConfig, RugezenLayer, RugezenMinGRU
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.loading import random_model
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    from tinyserve_llm_amd.ops import hip
    from tinyserve_llm_amd.parts.base import StepContext

    sizes = SHAPES[args.shape]
    sh = sizes["shape"]
    layers = args.layers or sizes["layers_full"]
    hidden, nh, nkv, hd, inter, vocab = (sh["hidden_size"], sh["num_attention_heads"], sh["num_key_value_heads"], sh["head_dim"],
                                         sh["intermediate_size"], sh["vocab_size"])
    llama = LlamaConfig(num_hidden_layers=layers, rope_scaling=RopeScaling(**{**ROPE, "factor": sizes["rope_factor"]}), **sh)
    att = RugezenAttention(heads=nh, kv_heads=nkv, dim=hd, vdim=hd, rot_dims=hd // 2, rot_base=1.0e6, scale=hd ** -0.5,
                           softcap=30.0)
    ff = 3 * inter // 2                  # two matrices of this width hold what the gated feed-forward's three hold
    rug = RugezenConfig(vocab=vocab, width=hidden, norm_eps=1e-6, residual_mult=0.6, layers=tuple(
        RugezenLayer("mingru", RugezenMinGRU(width=hidden), ff) if i % 4 == 2 else RugezenLayer("attention", att, ff)
        for i in range(layers)))
    prompt_len = args.context
    max_model_len = max(MAX_MODEL_LEN, prompt_len + 1024)
    rng = random.Random(0)
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def whole_engine(config) -> dict:
        model = random_model(config, 0, torch.bfloat16, "cuda:0")
        out = {"parameters": sum(t.numel() for t in (getattr(part, name) for layer in model.layers
                                                     for part in layer.parts().values() for name in part.param_specs()))}

        def engine(batch):
            pages = batch * -(-max_model_len // PAGE) + 2
            sc = SchedulerConfig(max_model_len=max_model_len, max_num_seqs=batch,
                                 max_num_batched_tokens=max(prompt_len, batch + 1) + batch, watermark=0.0)
            return LLM(None, sc, CacheConfig(block_size=PAGE, caching=False), dtype=torch.bfloat16, num_blocks=pages, seed=0,
                       model=model)
        llm = engine(1)
        times = []
        for r in range(3):
            llm.add_request([rng.randrange(vocab) for _ in range(prompt_len)], SamplingParams(max_tokens=1, temperature=0.0, ignore_eos=True))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            llm.step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        out["prefill_tok_s"] = prompt_len / min(times[1:])
        del llm
        for batch in (1, 8, 64):
            llm = engine(batch)
            sp = SamplingParams(max_tokens=max_model_len - prompt_len, temperature=0.0, ignore_eos=True)
            for _ in range(batch):
                llm.add_request([rng.randrange(vocab) for _ in range(prompt_len)], sp)
            while any(q.in_prefill or not q.output_token_ids for q in llm.scheduler.running + llm.scheduler.waiting):
                llm.step()
            for _ in range(6):
                llm.step()
            steps = 32
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                llm.step()
            torch.cuda.synchronize()
            out[f"decode_b{batch}_tok_s"] = batch * steps / (time.perf_counter() - t0)
            del llm
        del model
        torch.cuda.empty_cache()
        return out

    def replayed(fn, reps: int) -> float:
        fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            kept = fn()
        best = float("inf")
        for _ in range(reps):
            sweep.sum()
            begin.record()
            graph.replay()
            end.record()
            end.synchronize()
            best = min(best, 1e3 * begin.elapsed_time(end))
        del kept, graph
        return best

    overhead = []

    def timed(fn, reps: int = 5) -> float:
        """Microseconds of the best of `reps` replays of `fn` recorded into a graph (what the host does
        between launches is then not in the time), each after a sweep of the caches, less what the replay of
        a graph of one tiny kernel takes."""
        if not overhead:
            tiny = torch.zeros(64, dtype=torch.int32, device="cuda")
            overhead.append(replayed(lambda: tiny.add_(1), reps))
        return max(replayed(fn, reps) - overhead[0], 1e-3)

    sweep = torch.zeros(128 << 20, dtype=torch.int32, device="cuda")
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    bf = torch.bfloat16

    def context(starts, counts, pool_page):
        positions, seq_of, cu, tables = [], [], [0], []
        per = -(-max(a + b for a, b in zip(starts, counts)) // PAGE)
        for i, (s0, n) in enumerate(zip(starts, counts)):
            positions += list(range(s0, s0 + n))
            seq_of += [i] * n
            cu.append(cu[-1] + n)
            tables.append(list(range(i * per, (i + 1) * per)))
        ends = [a + b for a, b in zip(starts, counts)]
        ctx = StepContext(num_tokens=len(positions), num_seqs=len(starts), token_ids=dev([0] * len(positions)), positions=dev(positions),
                          seq_of_token=dev(seq_of), cu_seqlens=dev(cu), context_lens=dev(ends), state_slots=dev(list(range(len(starts)))),
                          slot_mapping=[], block_tables=[dev(tables)], host_cu_seqlens=cu, host_starts=list(starts),
                          host_context_lens=ends, host_state_slots=list(range(len(starts))), page_size=PAGE)
        slots = dev([tables[i][p // PAGE] * PAGE + p % PAGE for i, p in zip(seq_of, positions)])
        return ctx, slots, len(starts) * per * (PAGE // pool_page)

    def kernel_pairs() -> dict:
        pairs = {}
        pool_page = 32
        mfma = hip.measure_peaks()
        read_peak, mfma_peak = mfma["read_GBps"] * 1e9, mfma["mfma_bf16_TFLOPs"] * 1e12
        for label, starts, counts in (("prompt portion", [0], [prompt_len]), ("decoded tokens, batch 64", [prompt_len] * 64, [1] * 64)):
            ctx, slots, pages = context(starts, counts, pool_page)
            T = ctx.num_tokens
            k = torch.randn(pages, nkv, pool_page, hd, device="cuda").to(bf).permute(0, 2, 1, 3)
            v = torch.randn(pages, nkv, hd, pool_page, device="cuda").to(bf).permute(0, 3, 1, 2)
            q = torch.randn(T, nh, hd, device="cuda").to(bf)
            keys = sum(n * (s0 + (n + 1) / 2) for s0, n in zip(starts, counts))
            flops = 4 * nh * hd * keys
            nbytes = sum(s0 + n for s0, n in zip(starts, counts)) * 2 * nkv * hd * 2
            plain_us = timed(lambda: hip.paged_attention(q, k, v, ctx, 0, hd ** -0.5))
            general_us = timed(lambda: hip.paged_attention(q, k, v, ctx, 0, hd ** -0.5, softcap=30.0, sink=True))
            if T > 64:
                pairs[f"attention, {label}"] = {"llama_us": plain_us, "rugezen_us": general_us, "flops": flops,
                                                "llama_frac_of_mfma": flops / plain_us * 1e6 / mfma_peak,
                                                "rugezen_frac_of_mfma": flops / general_us * 1e6 / mfma_peak}
            else:
                pairs[f"attention, {label}"] = {"llama_us": plain_us, "rugezen_us": general_us, "bytes": nbytes,
                                                "llama_frac_of_read": nbytes / plain_us * 1e6 / read_peak,
                                                "rugezen_frac_of_read": nbytes / general_us * 1e6 / read_peak}
            # rotation and cache write: bfloat16 q|k|v rows in, against 32-bit rows in with the head norms
            row = (nh + 2 * nkv) * hd
            table = torch.randn(max_model_len, hd, device="cuda")
            freqs = torch.rand(hd // 4, dtype=torch.float64, device="cuda")
            qkv16, qkv32 = torch.randn(T, row, device="cuda").to(bf), torch.randn(T, row, device="cuda")
            us_a = timed(lambda: hip.rope_store(qkv16, table, ctx.positions, slots, k, v, nh, nkv, hd))
            us_b = timed(lambda: hip.qkv_finish(qkv32, freqs, ctx.positions, slots, k, v, nh, nkv, hd, hd, bf, qk_norm_eps=1e-5, v_norm_eps=1e-5))
            bytes_a, bytes_b = T * row * 2 * 2, T * row * (4 + 2)
            pairs[f"rotation and cache write, {label}"] = {"llama_us": us_a, "rugezen_us": us_b, "llama_bytes": bytes_a, "rugezen_bytes": bytes_b,
                                                           "llama_frac_of_read": bytes_a / us_a * 1e6 / read_peak,
                                                           "rugezen_frac_of_read": bytes_b / us_b * 1e6 / read_peak}
            # residual sum and norm: bfloat16 stream and one norm, against the 32-bit stream, two branches and two norms
            x16, r16 = (torch.randn(T, hidden, device="cuda").to(bf) for _ in range(2))
            w16 = torch.ones(hidden, device="cuda").to(bf)
            x32, a32, b32 = (torch.randn(T, hidden, device="cuda") for _ in range(3))
            us_a = timed(lambda: hip.rmsnorm(x16, w16, 1e-5, r16))
            us_b = timed(lambda: hip.stream_update_norm(x32, a32, b32, w16, 0.6, (w16, w16), 1e-6, out_dtype=bf))
            bytes_a, bytes_b = T * hidden * 2 * 4, T * hidden * (4 * 4 + 2 * 2)
            pairs[f"residual sum and norms, {label}"] = {"llama_us": us_a, "rugezen_us": us_b, "llama_bytes": bytes_a, "rugezen_bytes": bytes_b,
                                                         "llama_frac_of_read": bytes_a / us_a * 1e6 / read_peak,
                                                         "rugezen_frac_of_read": bytes_b / us_b * 1e6 / read_peak}
            gu, up, bias = torch.randn(T, 2 * inter, device="cuda").to(bf), torch.randn(T, ff, device="cuda"), torch.randn(ff, device="cuda").to(bf)
            us_a = timed(lambda: hip.silu_mul(gu))
            us_b = timed(lambda: hip.bias_activation(up, bias, "relu2", bf))
            bytes_a, bytes_b = T * inter * 2 * 3, T * ff * (4 + 2)
            pairs[f"feed-forward activation, {label}"] = {"llama_us": us_a, "rugezen_us": us_b, "llama_bytes": bytes_a, "rugezen_bytes": bytes_b,
                                                          "llama_frac_of_read": bytes_a / us_a * 1e6 / read_peak,
                                                          "rugezen_frac_of_read": bytes_b / us_b * 1e6 / read_peak}
            zxg, state = torch.randn(T, 3 * hidden, device="cuda"), torch.zeros(len(starts), hidden, device="cuda")
            us_b = timed(lambda: hip.mingru_scan(zxg, bias[:2 * hidden].contiguous() if ff >= 2 * hidden else None, state, ctx.cu_seqlens,
                                                 ctx.state_slots, max(counts), bf))
            bytes_b = T * hidden * (3 * 4 + 2)
            pairs[f"minGRU scan, {label}"] = {"rugezen_us": us_b, "rugezen_bytes": bytes_b, "rugezen_frac_of_read": bytes_b / us_b * 1e6 / read_peak}
        pairs["peaks"] = {"read_GBps": read_peak / 1e9, "mfma_bf16_TFLOPs": mfma_peak / 1e12}
        return pairs

    record = {"designs": {"llama": whole_engine(llama), "rugezen": whole_engine(rug)}, "kernels": kernel_pairs(),
              "config": {"shape": args.shape, "layers": layers, "hidden": hidden, "heads": nh, "kv_heads": nkv, "head_dim": hd,
                         "llama_intermediate": inter, "rugezen_ff": ff, "rugezen_mingru_every": 4, "vocab": vocab,
                         "context": prompt_len, "dtype": "bf16", "data": "synthetic uniform token ids, random weights"}}
    print(json.dumps(record))
    return 0


class DesignBench:
    """What the comparisons of two designs share: whole-engine throughput of a configuration with random weights,
    a kernel's time from replays of a graph with cold caches, and a packed step's context over pages of its own."""

    def __init__(self, vocab: int, prompt_len: int) -> None:
        import torch
        self.vocab, self.prompt_len = vocab, prompt_len
        self.max_model_len = max(MAX_MODEL_LEN, prompt_len + 1024)
        self.rng = random.Random(0)
        self.begin, self.end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        self.sweep = torch.zeros(128 << 20, dtype=torch.int32, device="cuda")
        self.overhead: list[float] = []

    def whole_engine(self, config) -> dict:
        import math

        import torch

        from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
        from tinyserve_llm_amd.engine.loading import random_model
        from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
        from tinyserve_llm_amd.engine.sequence import SamplingParams
        vocab, prompt_len, max_model_len, rng = self.vocab, self.prompt_len, self.max_model_len, self.rng
        model = random_model(config, 0, torch.bfloat16, "cuda:0")
        out = {"parameters": sum(math.prod(ps.shape) for name, ps in model.param_specs().items() if name.startswith("layers."))}

        def engine(batch):
            pages = batch * -(-max_model_len // PAGE) + 2
            sc = SchedulerConfig(max_model_len=max_model_len, max_num_seqs=batch,
                                 max_num_batched_tokens=max(prompt_len, batch + 1) + batch, watermark=0.0)
            return LLM(None, sc, CacheConfig(block_size=PAGE, caching=False), dtype=torch.bfloat16, num_blocks=pages, seed=0,
                       model=model)
        llm = engine(1)
        times = []
        for r in range(3):
            llm.add_request([rng.randrange(vocab) for _ in range(prompt_len)], SamplingParams(max_tokens=1, temperature=0.0, ignore_eos=True))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            llm.step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        out["prefill_tok_s"] = prompt_len / min(times[1:])
        del llm
        for batch in (1, 8, 64):
            llm = engine(batch)
            sp = SamplingParams(max_tokens=max_model_len - prompt_len, temperature=0.0, ignore_eos=True)
            for _ in range(batch):
                llm.add_request([rng.randrange(vocab) for _ in range(prompt_len)], sp)
            while any(q.in_prefill or not q.output_token_ids for q in llm.scheduler.running + llm.scheduler.waiting):
                llm.step()
            for _ in range(6):
                llm.step()
            steps = 32
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                llm.step()
            torch.cuda.synchronize()
            out[f"decode_b{batch}_tok_s"] = batch * steps / (time.perf_counter() - t0)
            del llm
        del model
        torch.cuda.empty_cache()
        return out

    def replayed(self, fn, reps: int) -> float:
        import torch
        fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            kept = fn()
        best = float("inf")
        for _ in range(reps):
            self.sweep.sum()
            self.begin.record()
            graph.replay()
            self.end.record()
            self.end.synchronize()
            best = min(best, 1e3 * self.begin.elapsed_time(self.end))
        del kept, graph
        return best

    def timed(self, fn, reps: int = 5) -> float:
        """Microseconds of the best replay of `fn` recorded into a graph, each after a sweep of the caches,
        less what the replay of a graph of one tiny kernel takes."""
        import torch
        if not self.overhead:
            tiny = torch.zeros(64, dtype=torch.int32, device="cuda")
            self.overhead.append(self.replayed(lambda: tiny.add_(1), reps))
        return max(self.replayed(fn, reps) - self.overhead[0], 1e-3)

    def context(self, starts, counts, pool_page):
        """(a packed step in which request i feeds `counts[i]` tokens from position `starts[i]` over pages of its own,
        its cache slots, the pool pages of `pool_page` tokens that takes)."""
        import torch

        from tinyserve_llm_amd.parts.base import StepContext
        dev = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
        positions, seq_of, cu, tables = [], [], [0], []
        per = -(-max(a + b for a, b in zip(starts, counts)) // PAGE)
        for i, (s0, n) in enumerate(zip(starts, counts)):
            positions += list(range(s0, s0 + n))
            seq_of += [i] * n
            cu.append(cu[-1] + n)
            tables.append(list(range(i * per, (i + 1) * per)))
        ends = [a + b for a, b in zip(starts, counts)]
        slots = dev([tables[i][p // PAGE] * PAGE + p % PAGE for i, p in zip(seq_of, positions)])
        ctx = StepContext(num_tokens=len(positions), num_seqs=len(starts), token_ids=dev([0] * len(positions)), positions=dev(positions),
                          seq_of_token=dev(seq_of), cu_seqlens=dev(cu), context_lens=dev(ends), state_slots=dev(list(range(len(starts)))),
                          slot_mapping=[slots], block_tables=[dev(tables)], host_cu_seqlens=cu, host_starts=list(starts),
                          host_context_lens=ends, host_state_slots=list(range(len(starts))), page_size=PAGE)
        return ctx, slots, len(starts) * per * (PAGE // pool_page)


def fanotar(args) -> int:
    """The Fanotar decoder beside the Rugezen decoder at the layer sizes of `--shape`: whole-engine
    throughput, and the like kernels of the two side by side. One JSON line."""
    import torch

    from tinyserve_llm_amd.config.fanotar import FanotarAttention, FanotarConfig, FanotarExperts, FanotarGatedUnit, FanotarLayer
    from tinyserve_llm_amd.config.rugezen import RugezenAttention, RugezenConfig, RugezenLayer
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.loading import random_model
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    from tinyserve_llm_amd.ops import hip
    from tinyserve_llm_amd.parts.base import StepContext
    from tinyserve_llm_amd.parts.linear import linear

    sizes = SHAPES[args.shape]
    sh = sizes["shape"]
    layers = args.layers or sizes["layers_full"]
    hidden, nh, nkv, hd, inter, vocab = (sh["hidden_size"], sh["num_attention_heads"], sh["num_key_value_heads"], sh["head_dim"],
                                         sh["intermediate_size"], sh["vocab_size"])
    window, taps, experts, top = 1024, 4, 16, 4
    eff, sff = inter // 8, inter // 2                 # four experts of an eighth and a shared half: one dense width per token
    ratt = RugezenAttention(heads=nh, kv_heads=nkv, dim=hd, vdim=hd, rot_dims=hd // 2, rot_base=1.0e6, scale=hd ** -0.5, softcap=30.0)
    rug = RugezenConfig(vocab=vocab, width=hidden, norm_eps=1e-6, residual_mult=0.6,
                        layers=tuple(RugezenLayer("attention", ratt, 3 * inter // 2) for _ in range(layers)))

    def fan_layer(i):
        att = FanotarAttention(heads=nh, kv_heads=nkv, dim=hd, vdim=hd, conv=taps, window=window, scale=hd ** -0.5, q_temp_coef=0.1,
                               q_temp_every=1024, kv_from=i - 1 if i % 4 == 3 else None)
        dense = FanotarGatedUnit(inter, 7.0)
        moe = FanotarExperts(experts=experts, top=top, scale=2.5, expert=FanotarGatedUnit(eff, 7.0), shared=FanotarGatedUnit(sff, 7.0))
        return FanotarLayer(att, moe if i % 2 else dense)
    fan = FanotarConfig(vocab=vocab, width=hidden, norm_eps=1e-6, embedding_scale=float(hidden) ** 0.5,
                        layers=tuple(fan_layer(i) for i in range(layers)))
    prompt_len = args.context
    bench = DesignBench(vocab, prompt_len)
    whole_engine, timed, context = bench.whole_engine, bench.timed, bench.context
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    bf = torch.bfloat16

    def kernel_pairs() -> dict:
        pairs = {}
        pool_page = 32
        peaks = hip.measure_peaks()
        read_peak, mfma_peak = peaks["read_GBps"] * 1e9, peaks["mfma_bf16_TFLOPs"] * 1e12
        slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / nh) for h in range(nh)], device="cuda")
        sinks = torch.randn(nh, device="cuda")
        for label, starts, counts in (("prompt portion", [0], [prompt_len]), ("decoded tokens, batch 64", [prompt_len] * 64, [1] * 64)):
            ctx, slots, pages = context(starts, counts, pool_page)
            T = ctx.num_tokens
            k = torch.randn(pages, nkv, pool_page, hd, device="cuda").to(bf).permute(0, 2, 1, 3)
            v = torch.randn(pages, nkv, hd, pool_page, device="cuda").to(bf).permute(0, 3, 1, 2)
            q = torch.randn(T, nh, hd, device="cuda").to(bf)
            gate = torch.randn(T, nh * hd, device="cuda")
            seen = lambda s0, n, w: sum(min(p + 1, w) if w else p + 1 for p in range(s0, s0 + n))
            keys_r = sum(seen(s0, n, 0) for s0, n in zip(starts, counts))
            keys_f = sum(seen(s0, n, window) for s0, n in zip(starts, counts))
            us_r = timed(lambda: hip.paged_attention(q, k, v, ctx, 0, hd ** -0.5, softcap=30.0, sink=True))
            us_f = timed(lambda: hip.paged_attention(q, k, v, ctx, 0, hd ** -0.5, window, sinks=sinks, slopes=slopes, gate=gate))
            us_f0 = timed(lambda: hip.paged_attention(q, k, v, ctx, 0, hd ** -0.5, window, sinks=sinks, slopes=slopes))
            if T > 64:
                fr, ff_ = 4 * nh * hd * keys_r, 4 * nh * hd * keys_f
                pairs[f"attention, {label}"] = {"rugezen_us": us_r, "fanotar_us": us_f, "fanotar_us_without_gate": us_f0,
                                                "rugezen_flops": fr, "fanotar_flops": ff_,
                                                "rugezen_frac_of_mfma": fr / us_r * 1e6 / mfma_peak,
                                                "fanotar_frac_of_mfma": ff_ / us_f * 1e6 / mfma_peak}
            else:
                br = sum(s0 + n for s0, n in zip(starts, counts)) * 2 * nkv * hd * 2
                bfan = sum(min(s0 + n, window) for s0, n in zip(starts, counts)) * 2 * nkv * hd * 2
                pairs[f"attention, {label}"] = {"rugezen_us": us_r, "fanotar_us": us_f, "fanotar_us_without_gate": us_f0,
                                                "rugezen_bytes": br, "fanotar_bytes": bfan,
                                                "rugezen_frac_of_read": br / us_r * 1e6 / read_peak,
                                                "fanotar_frac_of_read": bfan / us_f * 1e6 / read_peak}
            # between projection and cache: rotation and three head norms, against convolution, two head norms and the state
            row = (nh + 2 * nkv) * hd
            freqs = torch.rand(hd // 4, dtype=torch.float64, device="cuda")
            qkv32 = torch.randn(T, row + nh * hd, device="cuda")
            plain32 = qkv32[:, :row].contiguous()
            conv = torch.randn(row, taps, device="cuda")
            state = torch.zeros(len(starts), taps - 1, row, device="cuda")
            nw = torch.ones(hd, device="cuda")
            us_r = timed(lambda: hip.qkv_finish(plain32, freqs, ctx.positions, slots, k, v, nh, nkv, hd, hd, bf, qk_norm_eps=1e-5, v_norm_eps=1e-5))

            def finish():
                fused = hip.conv_moves_state(ctx)              # (steps of single tokens: the state moves on in the same launch)
                out = hip.conv_finish(qkv32, conv, state, ctx, slots, k, v, nh, nkv, hd, hd, bf, q_norm=nw, k_norm=nw, eps=1e-5,
                                      temp_coef=0.1, temp_every=1024, moves_state=fused)
                if not fused:
                    hip.conv_state_update(state, qkv32, ctx)
                return out
            us_f = timed(finish)
            nbytes = T * row * (4 + 2)
            pairs[f"between projection and cache, {label}"] = {"rugezen_us": us_r, "fanotar_us": us_f, "bytes": nbytes,
                                                               "rugezen_frac_of_read": nbytes / us_r * 1e6 / read_peak,
                                                               "fanotar_frac_of_read": nbytes / us_f * 1e6 / read_peak}
            # the stream's sum and norms: two branches and two RMS norms once a layer, against one branch through its norm and
            # one norm out, twice a layer
            w16 = torch.ones(hidden, device="cuda").to(bf)
            x32, a32, b32 = (torch.randn(T, hidden, device="cuda") for _ in range(3))
            norm = (torch.full((1,), 0.5, device="cuda"), torch.ones(hidden, device="cuda"), torch.zeros(hidden, device="cuda"))
            us_r = timed(lambda: hip.stream_update_norm(x32, a32, b32, None, 0.6, (w16, w16), 1e-6, out_dtype=bf))
            us_f = timed(lambda: hip.dyt_stream(x32, a32, norm, norm, bf))
            bytes_r, bytes_f = T * hidden * (4 * 4 + 2 * 2), T * hidden * (3 * 4 + 2)
            pairs[f"stream sum and norms, {label}"] = {"rugezen_us": us_r, "fanotar_us": us_f, "rugezen_bytes": bytes_r, "fanotar_bytes": bytes_f,
                                                       "fanotar_launches_a_layer": 2,
                                                       "rugezen_frac_of_read": bytes_r / us_r * 1e6 / read_peak,
                                                       "fanotar_frac_of_read": bytes_f / us_f * 1e6 / read_peak}
            rff = 3 * inter // 2
            up, bias, gu = torch.randn(T, rff, device="cuda"), torch.randn(rff, device="cuda").to(bf), torch.randn(T, 2 * inter, device="cuda")
            us_r = timed(lambda: hip.bias_activation(up, bias, "relu2", bf))
            us_f = timed(lambda: hip.capped_glu(gu, 7.0, 1.702, 1.0, bf))
            bytes_r, bytes_f = T * rff * (4 + 2), T * inter * (2 * 4 + 2)
            pairs[f"feed-forward activation, {label}"] = {"rugezen_us": us_r, "fanotar_us": us_f, "rugezen_bytes": bytes_r, "fanotar_bytes": bytes_f,
                                                          "rugezen_frac_of_read": bytes_r / us_r * 1e6 / read_peak,
                                                          "fanotar_frac_of_read": bytes_f / us_f * 1e6 / read_peak}
            # the experts' two products (routing and grouping beside them) against a dense feed-forward's two of the same
            # operations per token through `linear`
            x16 = torch.randn(T, hidden, device="cuda").to(bf)
            router, corr = torch.randn(experts, hidden, device="cuda") * 0.02, torch.zeros(experts, device="cuda")
            wgu = (torch.randn(experts, 2 * eff, hidden, device="cuda") * 0.02).to(bf)
            wd = (torch.randn(experts, hidden, eff, device="cuda") * 0.02).to(bf)
            dgu = (torch.randn(2 * top * eff, hidden, device="cuda") * 0.02).to(bf)
            dd = (torch.randn(hidden, top * eff, device="cuda") * 0.02).to(bf)
            ids, wts = hip.moe_route(x16, router, corr, top, 2.5)
            tile_rows = hip.moe_tile_rows(ids.numel(), experts, bf, (hidden, eff))
            grouped = hip.moe_group(ids, experts, tile_rows)
            us_route = timed(lambda: hip.moe_route(x16, router, corr, top, 2.5))
            us_group = timed(lambda: hip.moe_group(ids, experts, tile_rows))

            def products():
                unit = hip.moe_gemm(x16, wgu, grouped, bf, per_token=True, glu=(7.0, 1.702, 1.0))
                return hip.moe_combine(hip.moe_gemm(unit, wd, grouped, torch.float32, per_token=False), wts)

            def dense():
                unit = hip.capped_glu(linear(x16, dgu, out_dtype=torch.float32), 7.0, 1.702, 1.0, bf)
                return linear(unit, dd, out_dtype=torch.float32)
            us_f, us_d = timed(products), timed(dense)
            flops = 2 * T * top * 3 * eff * hidden
            touched = min(experts, T * top) * 3 * eff * hidden * 2
            rec = {"fanotar_us": us_f, "dense_of_equal_work_us": us_d, "routing_us": us_route, "grouping_us": us_group, "flops": flops,
                   "tile_rows": tile_rows}
            if T > 64:
                rec.update(fanotar_frac_of_mfma=flops / us_f * 1e6 / mfma_peak, dense_frac_of_mfma=flops / us_d * 1e6 / mfma_peak)
            else:
                rec.update(expert_bytes=touched, fanotar_frac_of_read=touched / us_f * 1e6 / read_peak,
                           dense_bytes=top * 3 * eff * hidden * 2, dense_frac_of_read=top * 3 * eff * hidden * 2 / us_d * 1e6 / read_peak)
            pairs[f"experts' products, {label}"] = rec
        pairs["peaks"] = {"read_GBps": read_peak / 1e9, "mfma_bf16_TFLOPs": mfma_peak / 1e12}
        return pairs

    record = {"designs": {"rugezen": whole_engine(rug), "fanotar": whole_engine(fan)}, "kernels": kernel_pairs(),
              "config": {"shape": args.shape, "layers": layers, "hidden": hidden, "heads": nh, "kv_heads": nkv, "head_dim": hd,
                         "rugezen_ff": 3 * inter // 2, "fanotar_dense_ff": inter, "fanotar_experts": experts, "fanotar_top": top,
                         "fanotar_expert_ff": eff, "fanotar_shared_ff": sff, "fanotar_window": window, "fanotar_conv_taps": taps,
                         "fanotar_layers": "dense and routed feed-forward in turn; every fourth layer reads the cache of the one before",
                         "vocab": vocab, "context": prompt_len, "dtype": "bf16",
                         "data": "synthetic uniform token ids, random weights"}}
    print(json.dumps(record))
    return 0


def bafarax_design(shape: str, layers: int | None):
    """The Bafarax configuration that `--bafarax` measures at the layer sizes of `shape`, and those sizes by name."""
    from tinyserve_llm_amd.config.bafarax import (BafaraxAttention, BafaraxConfig, BafaraxDense, BafaraxExperts, BafaraxLatentAttention,
                                                  BafaraxLayer, BafaraxMLSTM, FrequencyRamp, Rotation)
    sizes = SHAPES[shape]
    sh = sizes["shape"]
    layers = layers or sizes["layers_full"]
    hidden, nh, nkv, hd, inter, vocab = (sh["hidden_size"], sh["num_attention_heads"], sh["num_key_value_heads"], sh["head_dim"],
                                         sh["intermediate_size"], sh["vocab_size"])
    window, taps, experts, top = 1024, 4, 16, 4
    eff, sff = inter // 8, inter // 2
    # Bafarax: chunks as long as Fanotar's window; a latent of 256 with 32 turning dimensions beside heads of the shape's
    # size; a matrix memory of 8 heads whose values are twice as wide as its keys; four ungated experts of 3/8 of the dense
    # width each (two matrices where a gated unit has three): one dense width per token
    chunk, rank, q_rank, rot, bff = 1024, 256, 768, 32, 3 * inter // 8
    mh, md, mv = 8, hidden // 16, hidden // 8
    b_att = BafaraxAttention(heads=nh, kv_heads=nkv, dim=hd, vdim=hd, scale=hd ** -0.5, rot=Rotation(hd, 250000.0), chunk=chunk)
    b_lat = BafaraxLatentAttention(heads=nh, dim=hd, rot_dim=rot, vdim=hd, kv_rank=rank, q_rank=q_rank, scale=(hd + rot) ** -0.5,
                                   rot=Rotation(rot, 10000.0, FrequencyRamp(factor=8.0, original=4096.0, fast=32.0, slow=1.0)), window=window)
    b_mem = BafaraxMLSTM(heads=mh, dim=md, vdim=mv, gate_cap=15.0)
    b_moe, b_dense = BafaraxExperts(experts=experts, top=top, ff=bff), BafaraxDense(inter)
    cycle = (("attention", b_att, b_dense), ("latent_attention", b_lat, b_moe), ("mlstm", b_mem, b_dense), ("latent_attention", b_lat, b_moe))
    baf = BafaraxConfig(vocab=vocab, width=hidden, norm_eps=1e-6, embedding_scale=float(hidden) ** 0.5,
                        layers=tuple(BafaraxLayer(*cycle[i % 4]) for i in range(layers)))

    return baf, dict(layers=layers, hidden=hidden, nh=nh, nkv=nkv, hd=hd, inter=inter, vocab=vocab, window=window, taps=taps,
                     experts=experts, top=top, eff=eff, sff=sff, chunk=chunk, rank=rank, q_rank=q_rank, rot=rot, bff=bff, mh=mh, md=md, mv=mv)


def bafarax(args) -> int:
    """The Bafarax decoder beside the Fanotar decoder at the layer sizes of `--shape`: whole-engine throughput, and
    the like kernels of the two side by side. One JSON line."""
    import torch

    from tinyserve_llm_amd.config.fanotar import FanotarAttention, FanotarConfig, FanotarExperts, FanotarGatedUnit, FanotarLayer
    from tinyserve_llm_amd.ops import hip

    baf, z = bafarax_design(args.shape, args.layers)
    layers, hidden, nh, nkv, hd, inter, vocab = z["layers"], z["hidden"], z["nh"], z["nkv"], z["hd"], z["inter"], z["vocab"]
    window, taps, experts, top, eff, sff = z["window"], z["taps"], z["experts"], z["top"], z["eff"], z["sff"]
    chunk, rank, q_rank, rot, bff, mh, md, mv = z["chunk"], z["rank"], z["q_rank"], z["rot"], z["bff"], z["mh"], z["md"], z["mv"]

    def fan_layer(i):
        att = FanotarAttention(heads=nh, kv_heads=nkv, dim=hd, vdim=hd, conv=taps, window=window, scale=hd ** -0.5, q_temp_coef=0.1,
                               q_temp_every=1024, kv_from=i - 1 if i % 4 == 3 else None)
        moe = FanotarExperts(experts=experts, top=top, scale=2.5, expert=FanotarGatedUnit(eff, 7.0), shared=FanotarGatedUnit(sff, 7.0))
        return FanotarLayer(att, moe if i % 2 else FanotarGatedUnit(inter, 7.0))
    fan = FanotarConfig(vocab=vocab, width=hidden, norm_eps=1e-6, embedding_scale=float(hidden) ** 0.5,
                        layers=tuple(fan_layer(i) for i in range(layers)))
    prompt_len = args.context
    bench = DesignBench(vocab, prompt_len)
    timed, context = bench.timed, bench.context
    bf = torch.bfloat16

    def kernel_pairs() -> dict:
        pairs = {}
        pool_page = 32
        peaks = hip.measure_peaks()
        read_peak, mfma_peak, vector_peak = peaks["read_GBps"] * 1e9, peaks["mfma_bf16_TFLOPs"] * 1e12, PEAK_FLOPS["fp32"]
        slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / nh) for h in range(nh)], device="cuda")
        sinks = torch.randn(nh, device="cuda")
        row = rank + rot
        # (the decoded tokens stand in the middle of a chunk)
        for label, starts, counts in (("prompt portion", [0], [prompt_len]), ("decoded tokens, batch 64", [prompt_len + chunk // 2 - 1] * 64, [1] * 64)):
            ctx, slots, pages = context(starts, counts, pool_page)
            T, prompt = ctx.num_tokens, ctx.num_tokens > 64
            of_peak = lambda flops, nbytes, us: ({"frac_of_mfma": flops / us * 1e6 / mfma_peak} if prompt else
                                                 {"frac_of_read": nbytes / us * 1e6 / read_peak})
            k = torch.randn(pages, nkv, pool_page, hd, device="cuda").to(bf).permute(0, 2, 1, 3)
            v = torch.randn(pages, nkv, hd, pool_page, device="cuda").to(bf).permute(0, 3, 1, 2)
            q = torch.randn(T, nh, hd, device="cuda").to(bf)
            gate = torch.randn(T, nh * hd, device="cuda")
            spans = list(zip(starts, counts))
            seen_w = sum(min(p + 1, window) for s0, n in spans for p in range(s0, s0 + n))
            seen_c = sum(p % chunk + 1 for s0, n in spans for p in range(s0, s0 + n))
            # attention over the keys of the position's chunk with learned sinks, against a window, sinks, slopes and a gate
            us_f = timed(lambda: hip.paged_attention(q, k, v, ctx, 0, hd ** -0.5, window, sinks=sinks, slopes=slopes, gate=gate))
            us_b = timed(lambda: hip.paged_attention(q, k, v, ctx, 0, hd ** -0.5, 0, sinks=sinks, chunk_mask=chunk))
            pairs[f"attention in chunks, {label}"] = {
                "fanotar_us": us_f, "bafarax_us": us_b, "fanotar_keys": seen_w, "bafarax_keys": seen_c,
                "fanotar": of_peak(4 * nh * hd * seen_w, seen_w * 2 * nkv * hd * 2, us_f),
                "bafarax": of_peak(4 * nh * hd * seen_c, seen_c * 2 * nkv * hd * 2, us_b)}
            # attention through the latent: the keys' up-projection on the query's side, the turn of the queries' rotated
            # part, multi-query attention over the cached rows, the values' up-projection with the gate
            cache = torch.randn(pages, pool_page, 1, row, device="cuda").to(bf)
            values = cache[:, :, :, :rank].permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)      # transposed inside a page
            q32 = torch.randn(T, nh, hd + rot, device="cuda")
            uk = (torch.randn(nh, hd, rank, device="cuda") * 0.05).to(bf)
            uv = (torch.randn(nh, hd, rank, device="cuda") * 0.05).to(bf)
            uk_t = uk.transpose(1, 2).contiguous()           # (as the part keeps it: a head's dimensions along memory)
            freqs = torch.rand(rot // 2, dtype=torch.float64, device="cuda")
            absorbed = torch.empty(T, nh, row, device="cuda")
            heads = torch.empty(T, nh, hd, dtype=bf, device="cuda")

            def before():
                hip.heads_gemm(q32[:, :, :hd], uk_t.transpose(1, 2), absorbed[:, :, :rank])
                hip.rotate_heads(absorbed[:, :, rank:], q32[:, :, hd:], freqs, 1.2, ctx.positions, interleaved=True)
            before()
            attend = lambda: hip.paged_attention_latent(absorbed, cache, rank, ctx, 0, (hd + rot) ** -0.5, window, 0, out_dtype=bf, v_cache=values)
            mixed = attend()
            us_before = timed(before)
            us_att = timed(attend)
            us_after = timed(lambda: hip.heads_gemm(mixed, uv.transpose(1, 2), heads, gate=gate))
            flops_att = 2 * nh * seen_w * (row + rank)
            bytes_att = seen_w * (row + rank) * 2
            flops_heads = 2 * T * nh * hd * rank
            pairs[f"attention through a latent, {label}"] = {
                "fanotar_us": us_f, "bafarax_us": us_before + us_att + us_after, "bafarax_attention_us": us_att,
                "bafarax_products_before_us": us_before, "bafarax_product_after_us": us_after,
                "fanotar": of_peak(4 * nh * hd * seen_w, seen_w * 2 * nkv * hd * 2, us_f),
                "bafarax_attention": of_peak(flops_att, bytes_att, us_att),
                "bafarax_products": of_peak(2 * flops_heads, 2 * nh * hd * rank * 2 + T * nh * (row + rank) * 4, us_before + us_after)}
            # between projection and cache: a norm over the whole q and the whole k projection and the rotation; the latents'
            # norms and the shared key part's rotation; against the convolution, two head norms and its state
            qkv_row = (nh + 2 * nkv) * hd
            qkv32 = torch.randn(T, qkv_row + nh * hd, device="cuda")
            plain32 = qkv32[:, :qkv_row].contiguous()
            conv = torch.randn(qkv_row, taps, device="cuda")
            state = torch.zeros(len(starts), taps - 1, qkv_row, device="cuda")
            nw, qw, kw = torch.ones(hd, device="cuda"), torch.ones(nh * hd, device="cuda"), torch.ones(nkv * hd, device="cuda")
            rfreqs = torch.rand(hd // 2, dtype=torch.float64, device="cuda")

            def fan_finish():
                fused = hip.conv_moves_state(ctx)
                out = hip.conv_finish(qkv32, conv, state, ctx, slots, k, v, nh, nkv, hd, hd, bf, q_norm=nw, k_norm=nw, eps=1e-5,
                                      temp_coef=0.1, temp_every=1024, moves_state=fused)
                if not fused:
                    hip.conv_state_update(state, qkv32, ctx)
                return out

            def baf_finish():
                hip.segment_rmsnorm_pair(plain32, (0, nh * hd, qw), (nh * hd, nkv * hd, kw), 1e-6)
                return hip.qkv_finish(plain32, rfreqs, ctx.positions, slots, k, v, nh, nkv, hd, hd, bf, interleaved=False)
            down = torch.randn(T, q_rank + row + nh * hd, device="cuda")
            lqw, lcw = torch.ones(q_rank, device="cuda"), torch.ones(rank, device="cuda")
            us_f, us_b = timed(fan_finish), timed(baf_finish)
            us_l = timed(lambda: hip.latent_finish(down, 0, q_rank, q_rank, rank, rot, lqw, lcw, 1e-6, freqs, 1.2, ctx.positions, slots, cache, bf,
                                                   v_cache=values))
            nbytes, lbytes = T * qkv_row * (4 + 2), T * ((q_rank + row) * (4 + 2) + rank * 2)
            pairs[f"between projection and cache, {label}"] = {
                "fanotar_us": us_f, "bafarax_us": us_b, "bafarax_latent_us": us_l, "bytes": nbytes, "bafarax_latent_bytes": lbytes,
                "fanotar_frac_of_read": nbytes / us_f * 1e6 / read_peak, "bafarax_frac_of_read": nbytes / us_b * 1e6 / read_peak,
                "bafarax_latent_frac_of_read": lbytes / us_l * 1e6 / read_peak}
            # the stream's sum and the norm that reads it, twice a layer in both
            x32, a32 = torch.randn(T, hidden, device="cuda"), torch.randn(T, hidden, device="cuda")
            dyt = (torch.full((1,), 0.5, device="cuda"), torch.ones(hidden, device="cuda"), torch.zeros(hidden, device="cuda"))
            w32 = torch.ones(hidden, device="cuda")
            us_f = timed(lambda: hip.dyt_stream(x32, a32, dyt, dyt, bf))
            us_b = timed(lambda: hip.stream_update_norm(x32, a32, None, None, 1.0, (w32, None), 1e-6, out_dtype=bf))
            sbytes = T * hidden * (3 * 4 + 2)
            pairs[f"stream sum and norm, {label}"] = {"fanotar_us": us_f, "bafarax_us": us_b, "bytes": sbytes,
                                                      "fanotar_frac_of_read": sbytes / us_f * 1e6 / read_peak,
                                                      "bafarax_frac_of_read": sbytes / us_b * 1e6 / read_peak}
            # the experts: two products of ungated experts with a squared relu, against three of gated ones, equal work
            x16 = torch.randn(T, hidden, device="cuda").to(bf)
            router, corr = torch.randn(experts, hidden, device="cuda") * 0.02, torch.zeros(experts, device="cuda")
            wgu = (torch.randn(experts, 2 * eff, hidden, device="cuda") * 0.02).to(bf)
            wd = (torch.randn(experts, hidden, eff, device="cuda") * 0.02).to(bf)
            wup = (torch.randn(experts, bff, hidden, device="cuda") * 0.02).to(bf)
            wdn = (torch.randn(experts, hidden, bff, device="cuda") * 0.02).to(bf)
            ids, wts = hip.moe_route(x16, router, None, top, 1.0, True, softmax_chosen=True)
            tr_f, tr_b = hip.moe_tile_rows(ids.numel(), experts, bf, (hidden, eff)), hip.moe_tile_rows(ids.numel(), experts, bf, (hidden, bff))
            g_f, g_b = hip.moe_group(ids, experts, tr_f), hip.moe_group(ids, experts, tr_b)
            us_route_f = timed(lambda: hip.moe_route(x16, router, corr, top, 2.5))
            us_route_b = timed(lambda: hip.moe_route(x16, router, None, top, 1.0, True, softmax_chosen=True))

            def fan_products():
                unit = hip.moe_gemm(x16, wgu, g_f, bf, per_token=True, glu=(7.0, 1.702, 1.0))
                return hip.moe_combine(hip.moe_gemm(unit, wd, g_f, torch.float32, per_token=False), wts)

            def baf_products():
                act = hip.moe_gemm(x16, wup, g_b, bf, per_token=True, activation="relu2")
                return hip.moe_combine(hip.moe_gemm(act, wdn, g_b, torch.float32, per_token=False), wts)
            us_f, us_b = timed(fan_products), timed(baf_products)
            flops_f, flops_b = 2 * T * top * 3 * eff * hidden, 2 * T * top * 2 * bff * hidden
            touched_f, touched_b = min(experts, T * top) * 3 * eff * hidden * 2, min(experts, T * top) * 2 * bff * hidden * 2
            pairs[f"experts' products, {label}"] = {"fanotar_us": us_f, "bafarax_us": us_b, "fanotar_routing_us": us_route_f,
                                                    "bafarax_routing_us": us_route_b, "fanotar": of_peak(flops_f, touched_f, us_f),
                                                    "bafarax": of_peak(flops_b, touched_b, us_b)}
            # the matrix memory: the scan and what follows it; beside it the engine's other recurrence, a minGRU of the model's
            # width (a number per channel where this one keeps a matrix per head)
            width = 2 * mh * md + mh * mv + 2 * mh + mh * mv
            proj = torch.randn(T, width, device="cuda")
            gb = torch.zeros(2 * mh, device="cuda")
            mstate = torch.zeros(len(starts), hip.mlstm_state_size(mh, md, mv), device="cuda")
            mw = torch.ones(mh * mv, device="cuda")

            def memory():
                o = hip.mlstm_scan(proj, gb[:mh], gb[mh:], mstate, ctx.cu_seqlens, ctx.state_slots, mh, md, mv, 15.0,
                                   host_cu_seqlens=ctx.host_cu_seqlens, scratch=ctx.scratch)
                return hip.mlstm_finish(o, mw, proj[:, width - mh * mv:], mh, mv, 1e-6, bf)
            us_b = timed(memory)
            us_scan = timed(lambda: hip.mlstm_scan(proj, gb[:mh], gb[mh:], mstate, ctx.cu_seqlens, ctx.state_slots, mh, md, mv, 15.0,
                                                   host_cu_seqlens=ctx.host_cu_seqlens, scratch=ctx.scratch))
            zxg = torch.randn(T, 3 * hidden, device="cuda")
            gstate = torch.zeros(len(starts), hidden, device="cuda")
            us_g = timed(lambda: hip.mingru_scan(zxg, None, gstate, ctx.cu_seqlens, ctx.state_slots, max(counts), bf))
            mbytes = T * width * 4 + T * mh * mv * (4 + 4 + 2) + 2 * len(starts) * mstate.shape[1] * 4
            gbytes = T * hidden * (3 * 4 + 2) + 2 * len(starts) * hidden * 4
            mflops = 4 * T * mh * md * mv
            pairs[f"matrix memory, {label}"] = {"bafarax_us": us_b, "bafarax_scan_us": us_scan, "rugezen_mingru_us": us_g,
                                                "bafarax_bytes": mbytes, "rugezen_mingru_bytes": gbytes, "bafarax_flops_fp32": mflops,
                                                "bafarax_frac_of_read": mbytes / us_b * 1e6 / read_peak,
                                                "bafarax_frac_of_fp32_vector": mflops / us_b * 1e6 / vector_peak,
                                                "rugezen_mingru_frac_of_read": gbytes / us_g * 1e6 / read_peak}
        pairs["peaks"] = {"read_GBps": read_peak / 1e9, "mfma_bf16_TFLOPs": mfma_peak / 1e12, "fp32_vector_TFLOPs_published": vector_peak / 1e12}
        return pairs

    record = {"designs": {} if args.kernels_only else {"fanotar": bench.whole_engine(fan), "bafarax": bench.whole_engine(baf)},
              "kernels": kernel_pairs(),
              "config": {"shape": args.shape, "layers": layers, "hidden": hidden, "heads": nh, "kv_heads": nkv, "head_dim": hd,
                         "fanotar_window": window, "fanotar_experts": experts, "fanotar_top": top, "fanotar_expert_ff": eff,
                         "fanotar_shared_ff": sff, "bafarax_chunk": chunk, "bafarax_window": window, "bafarax_kv_rank": rank,
                         "bafarax_q_rank": q_rank, "bafarax_rot_dim": rot, "bafarax_expert_ff": bff,
                         "bafarax_memory": {"heads": mh, "dim": md, "vdim": mv},
                         "bafarax_layers": "in turn: attention in chunks with a dense feed-forward, latent attention with experts, "
                                           "a matrix memory with a dense feed-forward, latent attention with experts",
                         "vocab": vocab, "context": prompt_len, "dtype": "bf16",
                         "data": "synthetic uniform token ids, random weights"}}
    print(json.dumps(record))
    return 0


def tegolix_design(shape: str, layers: int | None):
    """The Tegolix configuration that `--tegolix` measures at the layer sizes of `shape`, and those sizes by name."""
    from tinyserve_llm_amd.config.bafarax import FrequencyRamp, Rotation
    from tinyserve_llm_amd.config.tegolix import (TegolixConfig, TegolixDense, TegolixExperts, TegolixGLA, TegolixLayer, TegolixParallel,
                                                  TegolixRecurrence, TegolixWindowAttention)
    sizes = SHAPES[shape]
    sh = sizes["shape"]
    layers = layers or sizes["layers_full"]
    hidden, nh, nkv, hd, inter, vocab = (sh["hidden_size"], sh["num_attention_heads"], sh["num_key_value_heads"], sh["head_dim"],
                                         sh["intermediate_size"], sh["vocab_size"])
    # gated linear attention of the matrix memory's sizes (8 heads, values twice as wide as keys); beside the windowed attention of
    # the shape's heads a recurrence of heads of 64; 16 gated experts of an eighth of the dense width and two identity experts, of
    # which a token uses 4, with a shared expert of half the dense width; 256 numbers of a second token table a layer
    window, experts, identity, top, eff, sff, side = 1024, 16, 2, 4, inter // 8, inter // 2, 256
    gh, gd, gv, rh, rd, rank = 8, hidden // 16, hidden // 8, hidden // 64, 64, 64
    gla = TegolixGLA(heads=gh, dim=gd, vdim=gv, tau=16.0, decay_rank=rank)
    left = TegolixWindowAttention(heads=nh, kv_heads=nkv, dim=hd, vdim=hd, scale=hd ** -0.5, softcap=30.0, window=window,
                                  rot=Rotation(hd // 2, 10000.0, FrequencyRamp(factor=8.0, original=4096.0, fast=32.0, slow=1.0)))
    par = TegolixParallel(left, TegolixRecurrence(heads=rh, dim=rd, decay_rank=rank), left_scale=0.6, right_scale=1.1)
    moe, dense = TegolixExperts(experts=experts, identity=identity, top=top, ff=eff, shared_ff=sff), TegolixDense(inter)
    cycle = (("gla", gla, dense), ("parallel", par, moe), ("gla", gla, dense), ("parallel", par, moe))
    teg = TegolixConfig(vocab=vocab, width=hidden, norm_eps=1e-6, side_dim=side, layers=tuple(TegolixLayer(*cycle[i % 4]) for i in range(layers)))
    return teg, dict(window=window, experts=experts, identity=identity, top=top, eff=eff, sff=sff, side=side, gh=gh, gd=gd, gv=gv, rh=rh, rd=rd, rank=rank)


def tegolix(args) -> int:
    """The Tegolix decoder beside the Bafarax decoder (the engine's closest design: a 32-bit stream with norms stored around
    zero, a matrix memory, windowed attention, experts) at the layer sizes of `--shape`: whole-engine throughput, and the like
    kernels of the two side by side. One JSON line."""
    import torch

    from tinyserve_llm_amd.ops import hip

    baf, z = bafarax_design(args.shape, args.layers)
    teg, t = tegolix_design(args.shape, args.layers)
    layers, hidden, nh, nkv, hd, vocab = z["layers"], z["hidden"], z["nh"], z["nkv"], z["hd"], z["vocab"]
    chunk, mh, md, mv = z["chunk"], z["mh"], z["md"], z["mv"]
    window, gh, gd, gv, rh, rd = t["window"], t["gh"], t["gd"], t["gv"], t["rh"], t["rd"]
    prompt_len = args.context
    bench = DesignBench(vocab, prompt_len)
    timed, context = bench.timed, bench.context
    bf = torch.bfloat16

    def kernel_pairs() -> dict:
        pairs = {}
        pool_page = 32
        peaks = hip.measure_peaks()
        read_peak, mfma_peak, vector_peak = peaks["read_GBps"] * 1e9, peaks["mfma_bf16_TFLOPs"] * 1e12, PEAK_FLOPS["fp32"]
        sinks = torch.randn(nh, device="cuda")
        for label, starts, counts in (("prompt portion", [0], [prompt_len]), ("decoded tokens, batch 64", [prompt_len + chunk // 2 - 1] * 64, [1] * 64)):
            ctx, slots, pages = context(starts, counts, pool_page)
            T, prompt, R = ctx.num_tokens, ctx.num_tokens > 64, len(starts)
            of_peak = lambda flops, nbytes, us: ({"frac_of_mfma": flops / us * 1e6 / mfma_peak} if prompt else
                                                 {"frac_of_read": nbytes / us * 1e6 / read_peak})
            k = torch.randn(pages, nkv, pool_page, hd, device="cuda").to(bf).permute(0, 2, 1, 3)
            v = torch.randn(pages, nkv, hd, pool_page, device="cuda").to(bf).permute(0, 3, 1, 2)
            q = torch.randn(T, nh, hd, device="cuda").to(bf)
            spans = list(zip(starts, counts))
            seen_w = sum(min(p + 1, window) for s0, n in spans for p in range(s0, s0 + n))
            seen_c = sum(p % chunk + 1 for s0, n in spans for p in range(s0, s0 + n))
            # attention in a window with capped scores, against attention in chunks with learned sinks: the same kernels
            us_t = timed(lambda: hip.paged_attention(q, k, v, ctx, 0, hd ** -0.5, window, softcap=30.0))
            us_b = timed(lambda: hip.paged_attention(q, k, v, ctx, 0, hd ** -0.5, 0, sinks=sinks, chunk_mask=chunk))
            pairs[f"attention, {label}"] = {
                "tegolix_us": us_t, "bafarax_us": us_b, "tegolix_keys": seen_w, "bafarax_keys": seen_c,
                "tegolix": of_peak(4 * nh * hd * seen_w, seen_w * 2 * nkv * hd * 2, us_t),
                "bafarax": of_peak(4 * nh * hd * seen_c, seen_c * 2 * nkv * hd * 2, us_b)}
            # between projection and cache: the heads' weighted norms, the values' turn, the rotation and the cache write, and after
            # attention the turn back with the gate per head; against the norms over the whole q and k and the rotation
            qkv_row = (nh + 2 * nkv) * hd
            qkv32 = torch.randn(T, qkv_row, device="cuda")
            nw, qw, kw = torch.ones(hd, device="cuda"), torch.ones(nh * hd, device="cuda"), torch.ones(nkv * hd, device="cuda")
            rfreqs = torch.rand(hd // 2, dtype=torch.float64, device="cuda")
            hfreqs = torch.rand(hd // 4, dtype=torch.float64, device="cuda")
            gate = torch.randn(T, nh, device="cuda")
            o16 = torch.randn(T, nh, hd, device="cuda").to(bf)

            def teg_finish():
                hip.qkv_prepare(qkv32, ctx.positions, nh, nkv, hd, hd, q_weight=nw, k_weight=nw, eps=1e-6, value_freqs=rfreqs)
                out = hip.qkv_finish(qkv32, hfreqs, ctx.positions, slots, k, v, nh, nkv, hd, hd, bf, interleaved=False, amplitude=1.2)
                hip.rotate_heads(o16, o16, rfreqs, 1.0, ctx.positions, interleaved=False, back=True, gate=gate)
                return out

            def baf_finish():
                hip.segment_rmsnorm_pair(qkv32, (0, nh * hd, qw), (nh * hd, nkv * hd, kw), 1e-6)
                return hip.qkv_finish(qkv32, rfreqs, ctx.positions, slots, k, v, nh, nkv, hd, hd, bf, interleaved=False)
            us_t, us_b = timed(teg_finish), timed(baf_finish)
            tbytes, bbytes = T * (qkv_row * (4 + 4 + 4 + 2) + nh * hd * 4), T * qkv_row * (4 + 4 + 4 + 2)
            pairs[f"between projection and cache, {label}"] = {
                "tegolix_us": us_t, "bafarax_us": us_b, "tegolix_bytes": tbytes, "bafarax_bytes": bbytes,
                "tegolix_frac_of_read": tbytes / us_t * 1e6 / read_peak, "bafarax_frac_of_read": bbytes / us_b * 1e6 / read_peak}
            # the stream's sum and the norm that reads it: with the branch's own norm and scale on the way in, against the sum alone
            x32, a32 = torch.randn(T, hidden, device="cuda"), torch.randn(T, hidden, device="cuda")
            w32 = torch.ones(hidden, device="cuda")
            us_t = timed(lambda: hip.stream_post_norm(x32, a32, w32, w32, 1e-6, w32, 1e-6, bf))
            us_b = timed(lambda: hip.stream_update_norm(x32, a32, None, None, 1.0, (w32, None), 1e-6, out_dtype=bf))
            sbytes = T * hidden * (3 * 4 + 2)
            pairs[f"stream sum and norm, {label}"] = {"tegolix_us": us_t, "bafarax_us": us_b, "bytes": sbytes,
                                                      "tegolix_frac_of_read": sbytes / us_t * 1e6 / read_peak,
                                                      "bafarax_frac_of_read": sbytes / us_b * 1e6 / read_peak}
            # the recurrences: gated linear attention (scan, then the heads' norm and gate) and the recurrence with token shift,
            # against the matrix memory at the gated linear attention's sizes
            gproj = torch.randn(T, 2 * gh * gd + 2 * gh * gv, device="cuda")
            gz, gbias, gnorm = torch.randn(T, gh * gd, device="cuda"), torch.full((gh * gd,), 3.0, device="cuda"), torch.ones(gv, device="cuda")
            gstate = torch.zeros(R, gh * gd * gv, device="cuda")
            K, V = gh * gd, gh * gv

            def gla():
                o = hip.decay_scan(gproj[:, :K], gproj[:, K:2 * K], gproj[:, 2 * K:2 * K + V], gz, gbias, gstate, ctx.cu_seqlens, ctx.state_slots,
                                   gh, gd, gv, form="sigmoid_root", tau=16.0, q_scale=gd ** -0.5, longest=max(counts))
                return hip.mlstm_finish(o, gnorm, gproj[:, 2 * K + V:], gh, gv, 1e-6, bf, silu_gate=True)
            us_gla = timed(gla)
            us_gla_scan = timed(lambda: hip.decay_scan(gproj[:, :K], gproj[:, K:2 * K], gproj[:, 2 * K:2 * K + V], gz, gbias, gstate, ctx.cu_seqlens,
                                                       ctx.state_slots, gh, gd, gv, form="sigmoid_root", tau=16.0, q_scale=gd ** -0.5, longest=max(counts)))
            rr, rk, rv, rg, rz = (torch.randn(T, rh * rd, device="cuda") for _ in range(5))
            rbias, rbonus, rnorm = torch.full((rh * rd,), -3.0, device="cuda"), torch.randn(rh, rd, device="cuda"), torch.ones(rh * rd, device="cuda")
            rstate = torch.zeros(R, rh * rd * rd + hidden, device="cuda")
            h16, mu = torch.randn(T, hidden, device="cuda").to(bf), torch.rand(5, hidden, device="cuda")

            def shifted():
                kept = rstate[:, rh * rd * rd:]
                mixes = hip.token_shift(h16, mu, kept, ctx)
                hip.token_shift_keep(kept, h16, ctx)
                o = hip.decay_scan(rr, rk, rv, rz, rbias, rstate, ctx.cu_seqlens, ctx.state_slots, rh, rd, rd, form="double_exponent", bonus=rbonus, longest=max(counts))
                return mixes, hip.mlstm_finish(o, rnorm, rg, rh, rd, 1e-6, bf, silu_gate=True)
            us_shift = timed(shifted)
            width = 2 * mh * md + mh * mv + 2 * mh + mh * mv
            proj = torch.randn(T, width, device="cuda")
            gb = torch.zeros(2 * mh, device="cuda")
            mstate = torch.zeros(R, hip.mlstm_state_size(mh, md, mv), device="cuda")
            mw = torch.ones(mh * mv, device="cuda")

            def memory():
                o = hip.mlstm_scan(proj, gb[:mh], gb[mh:], mstate, ctx.cu_seqlens, ctx.state_slots, mh, md, mv, 15.0,
                                   host_cu_seqlens=ctx.host_cu_seqlens, scratch=ctx.scratch)
                return hip.mlstm_finish(o, mw, proj[:, width - mh * mv:], mh, mv, 1e-6, bf)
            us_b = timed(memory)
            gbytes = T * (3 * K + 2 * V) * 4 + T * V * (4 + 4 + 2) + 2 * R * gstate.shape[1] * 4
            sbytes = T * (5 * rh * rd * 4 + hidden * 2 * 6 + rh * rd * (4 + 4 + 2)) + 2 * R * rstate.shape[1] * 4
            mbytes = T * width * 4 + T * mh * mv * (4 + 4 + 2) + 2 * R * mstate.shape[1] * 4
            gflops, sflops, mflops = 4 * T * gh * gd * gv, 4 * T * rh * rd * rd, 4 * T * mh * md * mv
            pairs[f"recurrence, {label}"] = {
                "tegolix_gla_us": us_gla, "tegolix_gla_scan_us": us_gla_scan, "tegolix_shifted_us": us_shift, "bafarax_memory_us": us_b,
                "tegolix_gla_bytes": gbytes, "tegolix_shifted_bytes": sbytes, "bafarax_memory_bytes": mbytes, "tegolix_gla_flops_fp32": gflops,
                "tegolix_shifted_flops_fp32": sflops, "bafarax_memory_flops_fp32": mflops,
                "tegolix_gla_frac_of_read": gbytes / us_gla * 1e6 / read_peak, "tegolix_shifted_frac_of_read": sbytes / us_shift * 1e6 / read_peak,
                "bafarax_memory_frac_of_read": mbytes / us_b * 1e6 / read_peak,
                "tegolix_gla_frac_of_fp32_vector": gflops / us_gla * 1e6 / vector_peak,
                "tegolix_shifted_frac_of_fp32_vector": sflops / us_shift * 1e6 / vector_peak,
                "bafarax_memory_frac_of_fp32_vector": mflops / us_b * 1e6 / vector_peak}
        pairs["peaks"] = {"read_GBps": read_peak / 1e9, "mfma_bf16_TFLOPs": mfma_peak / 1e12, "fp32_vector_TFLOPs_published": vector_peak / 1e12}
        return pairs

    record = {"designs": {} if args.kernels_only else {"bafarax": bench.whole_engine(baf), "tegolix": bench.whole_engine(teg)},
              "kernels": kernel_pairs(),
              "config": {"shape": args.shape, "layers": layers, "hidden": hidden, "heads": nh, "kv_heads": nkv, "head_dim": hd,
                         "tegolix": {k: v for k, v in t.items()},
                         "tegolix_layers": "in turn: gated linear attention with a dense feed-forward, windowed attention beside a recurrence "
                                           "with token shift, with experts",
                         "bafarax_memory": {"heads": mh, "dim": md, "vdim": mv}, "bafarax_chunk": chunk,
                         "vocab": vocab, "context": prompt_len, "dtype": "bf16", "data": "synthetic uniform token ids, random weights"}}
    print(json.dumps(record))
    return 0


def kernel_classes(llm, config, batch: int, reps: int = 5) -> dict:
    """Times one decode step's kernels by class. An eager step (no graph) is run once with every
    launch of the engine's kernel module noted down with its operands; then each class's launches
    (one per layer, with that layer's own weights) are recorded into a graph of their own, and the
    graph is replayed between two events after a sweep of the caches: a class's time is its kernels
    and the dispatches between them, as a recorded decode step sees them. Its bytes are what it has
    to read once (weights, or the keys and values of the live requests). The best of `reps` replays."""
    import torch

    from tinyserve_llm_amd.ops import hip

    c = config
    item = 2 if llm.dtype == torch.bfloat16 else 4
    by_shape = {(c.q_size + 2 * c.kv_size, c.hidden_size): "qkv", (c.hidden_size, c.q_size): "o",
                (2 * c.intermediate_size, c.hidden_size): "gate_up", (c.hidden_size, c.intermediate_size): "down",
                (c.vocab_size, c.hidden_size): "head"}
    calls: dict[str, list] = {}

    def note(klass, nbytes, inner, a, kw):
        calls.setdefault(klass, []).append((nbytes, inner, a, kw))
        return inner(*a, **kw)

    def product(name, weight_of):
        inner = getattr(hip, name)

        def noted(*a, **kw):
            w = weight_of(*a, **kw)
            if w.dim() == 4:                                   # a streaming copy: [N / 16, K / 32, 64, 8]
                shape = (w.shape[0] * 16, w.shape[1] * 32)
            elif w.dim() == 5:                                 # the 8-row form's: [N / 8, waves, steps, 64, 8]
                shape = (w.shape[0] * 8, w.shape[1] * w.shape[2] * 64)
            else:
                shape = tuple(w.shape)
            # (a copy's rows are padded to whole tiles)
            klass = next((v for k, v in by_shape.items() if k[1] == shape[1] and 0 <= shape[0] - k[0] < 16), f"product {shape}")
            return note(klass, shape[0] * shape[1] * item, inner, a, kw)
        return noted

    def other(name, klass, nbytes_of=lambda *a, **kw: 0):
        inner = getattr(hip, name)
        return lambda *a, **kw: note(klass, nbytes_of(*a, **kw), inner, a, kw)

    live = sum(s.num_tokens for s in llm.scheduler.running)
    kv_layer = live * 2 * c.kv_size * item
    patched = {
        "gemm_skinny": product("gemm_skinny", lambda x, w, *a, **kw: w),
        "gemm_skinny8": product("gemm_skinny8", lambda x, w, *a, **kw: w),
        "gemm_rows64": product("gemm_rows64", lambda x, packed, *a, **kw: packed),
        "gemm_rows64_sliced": product("gemm_rows64_sliced", lambda x, packed, *a, **kw: packed),
        "qkv_rope_store_sliced": product("qkv_rope_store_sliced", lambda x, packed, *a, **kw: packed),
        "gemm_library": product("gemm_library", lambda x, w, *a, **kw: w),
        "gemm_exact": product("gemm_exact", lambda x, w, *a, **kw: w),
        "qkv_rope_store": product("qkv_rope_store", lambda x, w, *a, **kw: w),
        "paged_attention_decode": other("paged_attention_decode", "attention", lambda *a, **kw: kv_layer),
        "paged_attention_wave": other("paged_attention_wave", "attention", lambda *a, **kw: kv_layer),
        "rmsnorm": other("rmsnorm", "norm"), "rope_store": other("rope_store", "rotation and cache write"),
        "silu_mul": other("silu_mul", "gate"), "sample": other("sample", "sampling"), "embedding": other("embedding", "embedding"),
    }
    kept = {name: getattr(hip, name) for name in patched}
    graphs, llm.runner.graphs, ahead = llm.runner.graphs, None, llm.run_ahead
    llm.run_ahead = False
    try:
        llm.step()                                         # (closes the step that was started ahead, starts none)
        for name, fn in patched.items():
            setattr(hip, name, fn)
        llm.step()
        torch.cuda.synchronize()
    finally:
        for name, fn in kept.items():
            setattr(hip, name, fn)
        llm.runner.graphs, llm.run_ahead = graphs, ahead
    sweep = torch.zeros(128 << 20, dtype=torch.int32, device="cuda")       # 512 MB: more than the caches hold
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    classes: dict[str, dict] = {}
    tiny = torch.zeros(64, dtype=torch.int32, device="cuda")
    calls = {"(a graph of one small kernel)": [(0, lambda: tiny.add_(1), (), {})], **calls}
    overhead = 0.0
    with torch.inference_mode():                          # (the step's tensors were made under it)
        for klass, noted in calls.items():
            for _, inner, a, kw in noted:                      # once outside a recording (libraries set themselves up)
                inner(*a, **kw)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                outs = [inner(*a, **kw) for _, inner, a, kw in noted]
            times = []
            for _ in range(reps + 1):
                sweep.sum()                                    # read, not written: the caches hold nothing of the weights, and nothing dirty
                begin.record()
                graph.replay()
                end.record()
                end.synchronize()
                times.append(1e3 * begin.elapsed_time(end))
            del outs, graph
            us, nbytes = max(min(times[1:]) - overhead, 1e-3), sum(n for n, *_ in noted)     # (a class of one tiny kernel may cost no more than the replay itself)
            if klass.startswith("("):
                overhead = us                                  # what a replay costs before its first kernel's work: taken off every class
                continue
            classes[klass] = {"launches": len(noted), "bytes": nbytes, "us": us, "us_per_launch": us / len(noted),
                              "GBps": nbytes / us / 1e3, "frac_of_hbm": nbytes / us * 1e6 / HBM_BYTES_PER_S}
    total = {"bytes": sum(r["bytes"] for r in classes.values()), "us": sum(r["us"] for r in classes.values())}
    total["GBps"] = total["bytes"] / total["us"] / 1e3
    return {"batch": batch, "live_tokens": live, "classes": dict(sorted(classes.items(), key=lambda kv: -kv[1]["us"])),
            "all_classes": total, "replay_overhead_us": overhead}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None)
    ap.add_argument("--shape", default="1b", choices=sorted(SHAPES), help="layer sizes of the decode and prefill steps")
    ap.add_argument("--context", type=int, default=PROMPT_LEN,
                    help="tokens of every prompt: the decode steps start from contexts of this length, and the prefill "
                         "is of this many tokens (the headline numbers are quoted at the default)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--points", default="1,64", help="further decode batch sizes (comma-separated; '' for none)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--only", default="all", choices=["all", "prefill"],
                    help="'prefill': time the 2,048-token prefill alone and print its record (for profiling)")
    ap.add_argument("--scenario", default=None, choices=sorted(SCENARIOS),
                    help="run a whole workload through LLM.generate instead of the decode step")
    ap.add_argument("--designs", action="store_true",
                    help="measure the Rugezen decoder beside the Llama decoder at the layer sizes of --shape: whole-engine "
                         "throughput and the like kernels side by side; one JSON line")
    ap.add_argument("--fanotar", action="store_true",
                    help="measure the Fanotar decoder beside the Rugezen decoder at the layer sizes of --shape: whole-engine "
                         "throughput and the like kernels side by side; one JSON line")
    ap.add_argument("--bafarax", action="store_true",
                    help="measure the Bafarax decoder beside the Fanotar decoder at the layer sizes of --shape: whole-engine "
                         "throughput and the like kernels side by side; one JSON line")
    ap.add_argument("--tegolix", action="store_true",
                    help="the Tegolix decoder beside the Bafarax decoder at the layer sizes of --shape: throughput and like kernels")
    ap.add_argument("--kernels-only", action="store_true", help="with --bafarax or --tegolix: the kernels side by side, no whole-engine runs")
    ap.add_argument("--kernel-classes", action="store_true",
                    help="time one decode step's kernels class by class (bytes, microseconds, GB/s) and exit")
    ap.add_argument("--peaks", action="store_true",
                    help="measure what a kernel that only reads memory and a loop of matrix instructions reach on "
                         "this GPU, print them beside the published peaks and exit")
    ap.add_argument("--many-rows-products", default="library", choices=["library", "tiled"],
                    help="bfloat16 products of many rows: the vendor's library, or the engine's own tiled kernel")
    args = ap.parse_args()
    if args.many_rows_products != "library":
        from tinyserve_llm_amd.ops import hip
        hip.many_rows_products(args.many_rows_products)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2
    if args.peaks:
        from tinyserve_llm_amd.ops import hip
        measured = hip.measure_peaks()
        print(json.dumps({"peaks": {"read": {"measured": measured["read_GBps"], "published": HBM_BYTES_PER_S / 1e9, "unit": "GB/s"},
                                    "mfma_bf16": {"measured": measured["mfma_bf16_TFLOPs"], "published": PEAK_FLOPS["bf16"] / 1e12,
                                                  "unit": "TFLOP/s"}}}))
        return 0
    if args.scenario:
        return scenario(args.scenario, args.layers, args.dtype)
    if args.designs:
        return designs(args)
    if args.fanotar:
        return fanotar(args)
    if args.bafarax:
        return bafarax(args)
    if args.tegolix:
        return tegolix(args)
    sizes = SHAPES[args.shape]
    full_layers = sizes["layers_full"]
    args.layers = args.layers or full_layers

    import torch

    from tinyserve_llm_amd.config import LlamaConfig, RopeScaling
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.loading import random_model
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams

    config = LlamaConfig(num_hidden_layers=args.layers, rope_scaling=RopeScaling(**{**ROPE, "factor": sizes["rope_factor"]}),
                         **sizes["shape"])
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    itemsize = 2 if args.dtype == "bf16" else 4
    model = random_model(config, 0, dtype, "cuda:0")
    rng = random.Random(0)

    c = config
    layer_weights = (c.q_size + 2 * c.kv_size) * c.hidden_size + c.hidden_size * c.q_size \
        + 3 * c.intermediate_size * c.hidden_size
    weight_bytes = (args.layers * layer_weights + c.vocab_size * c.hidden_size) * itemsize   # the head; the embedding reads rows
    kv_bytes_per_token = 2 * args.layers * c.kv_size * itemsize

    prompt_len = args.context
    max_model_len = max(MAX_MODEL_LEN, prompt_len + 1024)

    def engine(batch: int, steps: int) -> LLM:
        pages = batch * -(-max_model_len // PAGE) + 2
        sc = SchedulerConfig(max_model_len=max_model_len, max_num_seqs=max(batch, 1),
                             max_num_batched_tokens=max(prompt_len, batch + 1) + batch, watermark=0.0)
        return LLM(None, sc, CacheConfig(block_size=PAGE, caching=False), dtype=dtype, num_blocks=pages, seed=0,
                   model=model)

    def decode(batch: int, steps: int, warmup: int, classes: bool = False):
        """(seconds for `steps` decode steps, mean context length over them); with `classes`, the
        kernel classes of one such step instead."""
        llm = engine(batch, steps + warmup)
        sp = SamplingParams(max_tokens=max_model_len - prompt_len, temperature=0.0, ignore_eos=True)
        for _ in range(batch):
            llm.add_request([rng.randrange(c.vocab_size) for _ in range(prompt_len)], sp)
        while any(s.in_prefill or not s.output_token_ids for s in llm.scheduler.running + llm.scheduler.waiting):
            llm.step()
        for _ in range(warmup):
            llm.step()
        assert len(llm.scheduler.running) == batch and not llm.scheduler.waiting
        if classes:
            return kernel_classes(llm, c, batch)
        ctx0 = llm.scheduler.running[0].num_tokens
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            llm.step()
        torch.cuda.synchronize()
        seconds = time.perf_counter() - t0
        assert all(r.num_tokens == batch for r in llm.steps[-steps:])
        return seconds, ctx0 + (steps - 1) / 2

    def prefill(reps: int = 3) -> float:
        llm = engine(1, 1)
        sp = SamplingParams(max_tokens=1, temperature=0.0, ignore_eos=True)
        times = []
        for r in range(reps + 1):
            llm.add_request([rng.randrange(c.vocab_size) for _ in range(prompt_len)], sp)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            llm.step()
            torch.cuda.synchronize()
            if r:
                times.append(time.perf_counter() - t0)
            assert not llm.scheduler.has_unfinished()
        return min(times)

    def prefill_record() -> dict:
        t = prefill()
        T = prompt_len
        linear_flops = 2 * T * args.layers * layer_weights + 2 * c.vocab_size * c.hidden_size
        attn_flops = args.layers * 4 * c.q_size * T * (T + 1) / 2
        return {"value": T / t, "tokens": T, "ms": 1e3 * t, "frac": (linear_flops + attn_flops) / t / PEAK_FLOPS[args.dtype]}

    if args.only == "prefill":
        print(json.dumps({"prefill": prefill_record()}))
        return 0
    if args.kernel_classes:
        print(json.dumps({"kernel_classes": decode(args.batch, 1, args.warmup, classes=True),
                          "config": {"model": sizes["model"], "layers": args.layers, "context": prompt_len, "dtype": args.dtype}}))
        return 0

    from tinyserve_llm_amd.ops import hip
    measured = hip.measure_peaks()       # what this box gives a kernel that only reads, and a loop of matrix instructions
    read_peak = measured["read_GBps"] * 1e9
    mfma_peak = measured["mfma_bf16_TFLOPs"] * 1e12 if args.dtype == "bf16" else None

    seconds, mean_ctx = decode(args.batch, args.steps, args.warmup)
    value = args.batch * args.steps / seconds
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_bytes_per_token
    achieved = step_bytes / (seconds / args.steps)
    record = {
        "metric": f"decode tok/s at batch {args.batch} ({sizes['model']}, {prompt_len:,}-token contexts)",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": 1e3 * seconds / args.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic uniform token ids, random weights N(0,0.02)",
        "config": {"model": sizes["model"], "layers": args.layers, "layers_full": full_layers,
                   "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
                   "head_dim": c.head_dim, "intermediate": c.intermediate_size, "vocab": c.vocab_size,
                   "global_batch": args.batch, "prompt_len": prompt_len, "seq_len": max_model_len,
                   "page_size": PAGE, "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": achieved / HBM_BYTES_PER_S, "measured_peak": read_peak / 1e9,
                     "frac_of_measured": achieved / read_peak},
    }
    if not args.no_prefill:
        record["prefill"] = prefill_record()
        if mfma_peak:
            record["prefill"]["measured_peak_tflops"] = mfma_peak / 1e12
            record["prefill"]["frac_of_measured"] = record["prefill"]["frac"] * PEAK_FLOPS[args.dtype] / mfma_peak
    points, detail = {}, {}
    for b in [int(x) for x in args.points.split(",") if x.strip()]:
        k = max(16, min(args.steps, 64))
        s, ctx = decode(b, k, 4)
        points[f"decode_b{b}"] = b * k / s
        rate = (weight_bytes + b * ctx * kv_bytes_per_token) / (s / k)
        detail[f"decode_b{b}"] = {"tok_s": b * k / s, "ms_per_step": 1e3 * s / k, "frac": rate / HBM_BYTES_PER_S,
                                  "frac_of_measured": rate / read_peak}
    if points:
        record["points"] = points
        record["points_detail"] = detail
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
