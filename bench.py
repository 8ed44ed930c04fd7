"""Benchmark of the ReDrafter decode step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--extra-steps E] [--no-cpu-baseline]
    python bench.py --cpu-kernels      (per-kernel CPU baselines only; no GPU needed)

Workload (the configuration the headline metric is quoted on): random-init Vicuna-7B-shaped Llama
in bf16 (32 layers, hidden 4096, 32 heads, FFN 11008, vocab 32000) with a ReDrafter head (hidden
4096, exit_dim 8192, 2 residual blocks, recurrent state), weights N(0, 0.02) from a fixed seed;
batch 8, prompts of 500 token ids uniform over the vocabulary (pad id excluded), beam 45 x 5,
greedy, generation capped at 500 + 2048 tokens.  A step is one draft -> verify -> accept pass.

One JSON line on stdout: tokens/sec over the K timed steps (all eight sequences together), the
roofline entry of the dominant hand-written kernel (attn_mfma_kernel, timed with HIP events inside
the library while the timed region runs), and a CPU baseline: the torch restatement of the same
step (oracle/torch_path.py) timed on this machine's host cores on a bounded sample.  Beside the
headline, the same step at other points of its operating range, E timed steps each (`long_context`:
prompts of 1500 and 2500 tokens; `ragged_acceptance`: prompts of 1200 tokens with the acceptance
decision replaced by random accepted lengths, so that rows shift, accepted rows are appended and
the trees grow -- random-init models accept nothing by themselves; `ragged_prompts`: prompts of 500
to 2500 tokens in one batch, left-padded; `rope_attention_launches`: the
headline's step with the opt-in fused rotation + append + attention kernel against the default two;
`sampling`: speculative sampling at temperature 1 on the headline's models and prompts, and on the
Llama-2-13B shape at batch 16, prompt 256, beam 64 x 5 -- step time, synchronised stage times and
the event times of the kernels of the sampling path).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "ml-recurrent-drafter_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import torch  # noqa: E402

LLAMA_7B = dict(vocab_size=32000, hidden_size=4096, intermediate_size=11008, num_hidden_layers=32,
                num_attention_heads=32, num_key_value_heads=32, rms_norm_eps=1e-6, hidden_act="silu",
                pad_token_id=0, max_position_embeddings=2048)
DRAFTER_7B = dict(vocab_size=32000, hidden_size=4096, exit_dim=8192, num_draft_layers=2, rnn=True)
BATCH, PROMPT, NEW_TOKENS, WIDTH, LENGTH, SEED = 8, 500, 2048, 45, 5, 123
MFMA_BF16_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0
TIMED_EVERY = 5  # the dominant kernel's launches are event-timed one in five
CPU_STEPS = 3  # timed steps per layer count of the CPU baseline


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# configuration 5 of the benchmark plan: Llama-2-13B shape, batch 16, prompt 256, beam 64 x 5, T = 1
LLAMA_13B = dict(LLAMA_7B, hidden_size=5120, intermediate_size=13824, num_hidden_layers=40,
                 num_attention_heads=40, num_key_value_heads=40)
DRAFTER_13B = dict(DRAFTER_7B, hidden_size=5120, exit_dim=10240)


def build_models(device: str, dtype: torch.dtype, n_layers: int, seed: int, llama_cfg=None, drafter_cfg=None):
    """Random-init pair; every weight N(0, 0.02) from one seeded generator, norm gains 1."""
    import recurrent_drafting_amd as rd
    from transformers.models.llama.configuration_llama import LlamaConfig

    llama_cfg, drafter_cfg = llama_cfg or LLAMA_7B, drafter_cfg or DRAFTER_7B
    prev = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        with torch.device(device):
            llm = rd.modeling_llama.LlamaForCausalLM(LlamaConfig(**dict(llama_cfg, num_hidden_layers=n_layers)))
            drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(**drafter_cfg))
    finally:
        torch.set_default_dtype(prev)
    gen = torch.Generator(device=device).manual_seed(seed)
    with torch.no_grad():
        for module in (llm, drafter):
            for name, p in sorted(module.named_parameters()):
                if name.endswith("layernorm.weight") or name.endswith("norm.weight"):
                    p.fill_(1.0)
                else:
                    p.normal_(0.0, 0.02, generator=gen)
    return llm.eval(), drafter.eval()


def prompts(device: str, length: int = PROMPT, batch: int = BATCH) -> torch.Tensor:
    gen = torch.Generator(device="cpu").manual_seed(SEED)
    return torch.randint(1, LLAMA_7B["vocab_size"], (batch, length), generator=gen).to(device)


# -------------------------------------------------------------------------------------------------
# GPU run
# -------------------------------------------------------------------------------------------------
def forced_acceptance(seed: int):
    """Stand-in for the acceptance decision: random accepted lengths (0 .. length-1) and beams per
    row and step.  Random-init models never accept a drafted token, so with the real decision the
    rows never shift, nothing is appended behind a prompt of ragged length and the trees stay at
    their smallest; this puts those paths into the timed region.  The tokens then mean nothing."""
    gen = torch.Generator().manual_seed(seed)

    def force(real):
        def accept(beams, llm_tokens, unpacker=None):
            n, s, nxt, last = real(beams, llm_tokens, unpacker)
            B, W, L = beams.shape
            n = torch.randint(0, L, (B,), generator=gen).to(beams.device)
            s = torch.randint(0, W, (B,), generator=gen).to(beams.device)
            rows = torch.arange(B, device=beams.device)
            last = unpacker[rows, s, n] if unpacker is not None else s * L + n
            nxt = llm_tokens[rows, last] if unpacker is not None else llm_tokens.reshape(B, -1)[rows, last]
            return n, s, nxt, last
        return accept
    return force


def timed_decode(model, ids, steps: int, warmup: int, max_new: int, force=None, temperature=None,
                 beam=(WIDTH, LENGTH)):
    """Runs warmup + steps decode steps of one generation (a new one is started, prefill untimed,
    whenever the cap is reached) and returns the timing of the `steps` steps, the shapes of the
    attention launches in them and the HIP-event time of every TIMED_EVERY-th of those launches.
    temperature None: greedy; a number: speculative sampling at that temperature."""
    import recurrent_drafting_amd as rd
    from recurrent_drafting_amd import _hip, acceptance, attention

    max_length = ids.shape[1] + max_new
    real_accept = acceptance.greedy_accept
    if force is not None:
        acceptance.greedy_accept = force(real_accept)
    try:
        ledger = rd.stats.Ledger(sync=False)

        def new_stream():
            sampling = rd.SamplingArgs(1.0, True) if temperature is None else rd.SamplingArgs(float(temperature), False)
            return model.generate(ledger, ids, max_length, rd.BeamShape(*beam), sampling, rd.SpecialTokens(0, None))

        stream = new_stream()
        for _ in range(warmup):
            next(stream)
        torch.cuda.synchronize()
        # HIP events around the launches of the dominant kernel, live in the timed region: every
        # TIMED_EVERY-th launch in launch order (the two events of a launch keep the GPU idle for about
        # 11 us; around all 32 launches of a step that is 2.4 % of the step, around every fifth 0.5 %;
        # five is coprime to the 32 layers, so the sample walks through the layers).
        shapes = []
        attention.shape_log = shapes
        _hip.timing_select("attn_mfma_kernel")
        _hip.timing_sample(TIMED_EVERY)
        _hip.timing_enable(True)
        elapsed, timed = 0.0, 0
        first_len = last_len = first_out = None
        out = None
        while timed < steps:
            torch.cuda.synchronize()
            start = time.perf_counter()
            seg, exhausted = 0, False
            while timed + seg < steps:
                try:
                    out = next(stream)
                except StopIteration:
                    exhausted = True
                    break
                seg += 1
                if first_len is None:
                    first_len, first_out = out.shape[1], out
                last_len = out.shape[1]
            torch.cuda.synchronize()
            elapsed += time.perf_counter() - start
            timed += seg
            if exhausted:  # generation reached its cap: start another one (prefill is not timed)
                stream = new_stream()
                for _ in range(warmup):
                    next(stream)
        dominant = _hip.timing_collect()
        _hip.timing_enable(False)
        _hip.timing_select(None)
        _hip.timing_sample(1)
        attention.shape_log = None
        left_pads = lambda ids: int((ids == 0).long().cumprod(dim=-1).sum())  # noqa: E731
        final_pads = left_pads(out) if out is not None else 0
        first_pads = left_pads(first_out) if first_out is not None else 0
        stream.close()  # posts the open generation's record
    finally:
        acceptance.greedy_accept = real_accept
    accepted = [a for rec in ledger.records for a in rec.get("avg_num_accepted", [])]
    per_seq_tokens = sum(a + 1 for a in accepted) / max(len(accepted), 1)
    cfg = model.llm.config
    return dict(elapsed=elapsed, steps=timed, per_seq_tokens=per_seq_tokens, tokens=per_seq_tokens * ids.shape[0] * timed,
                dominant=dominant, shapes=shapes, context=(first_len, last_len), final_left_pads=final_pads,
                first_left_pads=first_pads, heads=cfg.num_attention_heads,
                head_dim=cfg.hidden_size // cfg.num_attention_heads)


def synchronised_steps(model, ids, max_length, beam, temperature, warm: int = 2, steps: int = 4):
    """A few steps under the reference's synchronised stage timers, with every kernel of the library
    event-timed: -> (mean seconds per stage, {kernel: (launches, total ms)}, the ledger)."""
    import recurrent_drafting_amd as rd
    from recurrent_drafting_amd import _hip

    ledger = rd.stats.Ledger(sync=True)
    sampling = rd.SamplingArgs(1.0, True) if temperature is None else rd.SamplingArgs(float(temperature), False)
    stream = model.generate(ledger, ids, max_length, rd.BeamShape(*beam), sampling, rd.SpecialTokens(0, None))
    for _ in range(warm):
        next(stream)
    _hip.timing_enable(True)
    for _ in range(steps):
        next(stream)
    torch.cuda.synchronize()
    kernels = _hip.timing_collect()
    _hip.timing_enable(False)
    stream.close()
    rec = ledger.records[0]
    for key in ("step", "input_id_length", "avg_num_accepted"):  # drop the warm-up steps
        rec[key] = rec[key][warm:]
    rec["wall_times"] = {k: v[warm:] for k, v in rec["wall_times"].items()}
    stage = {k: sum(v) / len(v) for k, v in rec["wall_times"].items()}
    return stage, kernels, ledger


def sampling_point(model, ids, extra_steps: int, warmup: int, beam):
    """Speculative sampling at temperature 1 on the given models and prompts: the free-running step
    time, then the synchronised stage times and the kernels of the sampling path on a few more steps."""
    run = timed_decode(model, ids, extra_steps, warmup, 64 + 5 * (extra_steps + warmup), temperature=1.0, beam=beam)
    stage, kernels, _ = synchronised_steps(model, ids, ids.shape[1] + 64, beam, 1.0)
    run.update(stage=stage, kernels=kernels)
    return run


def gpu_run(steps: int, warmup: int, extra_steps: int):
    import recurrent_drafting_amd as rd
    from recurrent_drafting_amd import _hip

    dev = "cuda:0"
    t0 = time.perf_counter()
    llm, drafter = build_models(dev, torch.bfloat16, LLAMA_7B["num_hidden_layers"], SEED)
    torch.cuda.synchronize()
    log(f"[bench] models on {torch.cuda.get_device_name(0)} in {time.perf_counter() - t0:.1f}s")
    model = rd.RecurrentDrafting(llm, drafter)
    n_tuned = rd.gemm_tuning.load()  # opt-in kernel selection table for the dense layers' GEMMs (look-up only)
    log(f"[bench] GEMM kernel selection table: {n_tuned} entries in effect")

    # ---- the headline: prompt 500, generation capped at 2048 new tokens ------------------------------
    run = timed_decode(model, prompts(dev, PROMPT), steps, warmup, NEW_TOKENS)
    run["null_us"] = _hip.timing_null_kernel_us(64)

    # ---- the same step further along the trajectory, and with rows that accept drafted tokens -------
    others = {}
    if extra_steps > 0:
        for name, prompt_len, force in (("context_1500", 1500, None), ("context_2500", 2500, None),
                                        ("ragged_acceptance_context_1200", 1200, forced_acceptance(SEED))):
            r = timed_decode(model, prompts(dev, prompt_len), extra_steps, warmup, 64 + 5 * (extra_steps + warmup), force)
            r["null_us"] = run["null_us"]
            others[name] = r
            log(f"[bench] {name}: {r['elapsed'] / r['steps'] * 1e3:.2f} ms/step over {r['steps']} steps, "
                f"context {r['context']}, {r['per_seq_tokens']:.2f} tokens per sequence and step")
        # prompts of different lengths, left-padded to the longest, as a batch of unrelated requests
        # has them: the attention's rows then differ in their number of keys and its work items
        # are cut by the plan's model of the launch
        ids = prompts(dev, 2500)
        lens = torch.randint(500, 2501, (BATCH,), generator=torch.Generator().manual_seed(SEED))
        lens[0] = 2500
        for b, n in enumerate(lens.tolist()):
            ids[b, : 2500 - n] = 0
        r = timed_decode(model, ids, extra_steps, warmup, 64 + 5 * (extra_steps + warmup))
        r["null_us"] = run["null_us"]
        r["prompt_tokens"] = sorted(lens.tolist())
        others["prompts_of_500_to_2500_tokens"] = r
        log(f"[bench] prompts of {r['prompt_tokens']} tokens: {r['elapsed'] / r['steps'] * 1e3:.2f} ms/step")
        # rotation + cache append + attention of a layer as two launches (the default, and what every
        # other figure of this line is measured on) against one (rd_rope_verify_attention), back to
        # back on the headline's prompts
        from recurrent_drafting_amd import modeling_llama
        default = modeling_llama.LlamaAttention.fused_rope_attention
        try:
            for name, fused in (("two_kernels", False), ("one_kernel", None)):
                modeling_llama.LlamaAttention.fused_rope_attention = fused
                r = timed_decode(model, prompts(dev, PROMPT), extra_steps, warmup, 64 + 5 * (extra_steps + warmup))
                r["null_us"] = run["null_us"]
                others["rope_attention_" + name] = r
                log(f"[bench] rope + append + attention as {name}: {r['elapsed'] / r['steps'] * 1e3:.2f} ms/step")
        finally:
            modeling_llama.LlamaAttention.fused_rope_attention = default

        # speculative sampling at temperature 1 on the headline's models and prompts (the kernels of
        # recurrent_drafting.py:75-111, :499-556: row statistics of the packed logits, acceptance,
        # residual distribution; the float32 log-probability history of the drafter)
        r = sampling_point(model, prompts(dev, PROMPT), extra_steps, warmup, (WIDTH, LENGTH))
        r["null_us"] = run["null_us"]
        others["sampling_temperature_1"] = r
        log(f"[bench] sampling at temperature 1: {r['elapsed'] / r['steps'] * 1e3:.2f} ms/step, "
            f"{r['per_seq_tokens']:.2f} tokens per sequence and step")

    # ---- stage breakdown with the reference's synchronised timers, on a few extra steps ---------------
    stage, kernels, ledger2 = synchronised_steps(model, prompts(dev, PROMPT), PROMPT + NEW_TOKENS, (WIDTH, LENGTH), None)
    table, _ = rd.stats.summarize(ledger2, BATCH, LENGTH - 1)  # the reference's own summary (stats.py:158-215)
    run.update(kernels=kernels, stage=stage, ref_style_tokens_per_second=table.tokens_per_second, others=others)
    del model, llm, drafter
    torch.cuda.empty_cache()

    # ---- configuration 5: Llama-2-13B shape, batch 16, prompt 256, beam 64 x 5, sampling at T = 1 -------
    if extra_steps > 0:
        t0 = time.perf_counter()
        llm, drafter = build_models(dev, torch.bfloat16, LLAMA_13B["num_hidden_layers"], SEED + 1, LLAMA_13B, DRAFTER_13B)
        model = rd.RecurrentDrafting(llm, drafter)
        torch.cuda.synchronize()
        log(f"[bench] 13B-shaped models in {time.perf_counter() - t0:.1f}s")
        r = sampling_point(model, prompts(dev, 256, batch=16), extra_steps, warmup, (64, 5))
        r["null_us"] = run["null_us"]
        others["llama_13b_shape_batch_16_beam_64x5_sampling"] = r
        log(f"[bench] 13B shape, batch 16, beam 64x5, sampling: {r['elapsed'] / r['steps'] * 1e3:.2f} ms/step")
        del model, llm, drafter
        torch.cuda.empty_cache()
    return run


def attention_roofline(run):
    """The dominant kernel against the roof that binds it.  Per launch, from the shapes the timed
    region actually ran: algorithmic FLOPs 4 * heads * head_dim * query rows * keys, algorithmic
    bytes K and V once (2 * heads * head_dim * 2 B per key) plus Q and O once, query rows = the
    tree slots that exist (the padding slots of the (batch, n_q) layout are not run), keys = the
    keys between a row's left padding and its last tree slot; duration = HIP events around every
    TIMED_EVERY-th launch of the timed region (the shapes are those of the same launches).
    Arithmetic intensity below the machine balance (2500 TFLOP/s / 8 TB/s = 312 FLOP/B) means the
    HBM roof binds, above it the MFMA roof."""
    H, D = run.get("heads", LLAMA_7B["num_attention_heads"]), run.get("head_dim", 128)
    count, total_ms = run["dominant"].get("attn_mfma_kernel", (0, 0.0))
    launched = len(run["shapes"])
    shapes = run["shapes"][::TIMED_EVERY][:count] if count else []  # the launches that were timed
    if not count or total_ms <= 0:
        return None
    # keys: every row from its first real token to its last tree slot.  Left padding appears with
    # prompts of different lengths and with forced acceptance (rows grow at different rates); its
    # average over the run is taken as the mean of what the first and the last timed step show,
    # and the tree slots a row does not have are left out.
    pads = (run.get("first_left_pads", 0) + run.get("final_left_pads", 0)) / 2.0
    keys = [B * (kv - n_q) - pads + rows for (B, n_q, kv, rows) in shapes]
    flops = sum(4.0 * H * D * (rows / B) * k for (B, n_q, kv, rows), k in zip(shapes, keys))
    k_bytes = sum(2.0 * H * D * 2 * k + 2.0 * rows * H * D * 2 for (B, n_q, kv, rows), k in zip(shapes, keys))
    seconds = total_ms * 1e-3
    tflops, gbs = flops / seconds / 1e12, k_bytes / seconds / 1e9
    hbm_bound = flops / k_bytes < MFMA_BF16_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9)
    out = dict(kernel="attn_mfma_kernel")
    if hbm_bound:
        out.update(bound="hbm", achieved=round(gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(gbs / HBM_PEAK_GBS, 4))
    else:
        out.update(bound="mfma", achieved=round(tflops, 2), peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s",
                   frac=round(tflops / MFMA_BF16_PEAK_TFLOPS, 4))
    # HBM bytes by counters belong to the run they were counted on, not to this one: the figure of
    # this run is null, and the ratio (counted / algorithmic bytes) of the profiled run is named
    profiled = None
    path = os.path.join(ROOT, "profiles", "attn_mfma_kernel_traffic.json")
    if os.path.exists(path):
        with open(path) as f:
            j = json.load(f)
        profiled = dict(ratio=j.get("ratio"), workload=j.get("workload"))
    out.update(
        traffic=None, traffic_ratio_profiled=profiled,
        launches=count, launches_in_timed_region=launched, timed_every=TIMED_EVERY,
        avg_us=round(total_ms * 1e3 / count, 2),
        algorithmic_gflop_per_launch=round(flops / count / 1e9, 3),
        algorithmic_mb_per_launch=round(k_bytes / count / 1e6, 2),
        flop_per_byte=round(flops / k_bytes, 1),
        mfma_frac_of_peak=round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
        hbm_frac_of_peak=round(gbs / HBM_PEAK_GBS, 4),
        # HIP events span dispatch and completion signalling too; an empty kernel timed the same way
        # gives that fixed part (a kernel trace reports about avg_us minus this)
        null_kernel_event_us=round(run["null_us"], 2),
        mean_n_q=round(sum(n for (_, n, _, _) in shapes) / len(shapes), 1),
        mean_query_rows=round(sum(r for (_, _, _, r) in shapes) / len(shapes), 1),
        mean_kv_len=round(sum(kv for (_, _, kv, _) in shapes) / len(shapes), 1),
    )
    return out


SAMPLING_KERNELS = ("row_stats_kernel", "accept_sample_kernel", "residual_probs_kernel", "gather_rows_kernel",
                    "beam_row_kernel", "beam_merge_kernel", "attn_mfma_kernel")


def sampling_summary(run):
    """A sampling operating point: summary_of plus the synchronised times of the sampling-only stages
    and the event times of the kernels on the sampling path."""
    out = summary_of(run)
    out["stage_seconds_synchronised"] = {k: round(v, 6) for k, v in run["stage"].items()}
    out["kernel_avg_us"] = {k: round(ms * 1e3 / n, 2) for k, (n, ms) in sorted(run["kernels"].items())
                            if k in SAMPLING_KERNELS and n}
    return out


def summary_of(run):
    """One of the additional operating points: step time, throughput, the attention kernel."""
    r = attention_roofline(run)
    return dict(
        ms_per_step=round(run["elapsed"] / run["steps"] * 1e3, 3), steps=run["steps"],
        tokens_per_second=round(run["tokens"] / run["elapsed"], 2),
        tokens_per_step_per_sequence=round(run["per_seq_tokens"], 3),
        context_tokens=list(run["context"]),
        attention=None if r is None else {k: r[k] for k in (
            "avg_us", "bound", "achieved", "unit", "frac", "mfma_frac_of_peak", "algorithmic_mb_per_launch",
            "mean_n_q", "mean_query_rows", "mean_kv_len", "launches")},
    )


# -------------------------------------------------------------------------------------------------
# CPU baseline: the torch restatement of one step on the host cores, bounded sample
# -------------------------------------------------------------------------------------------------
def cpu_baseline(per_seq_tokens: float):
    from oracle import torch_path as P

    threads = torch.get_num_threads()
    a = torch.randn(1448, 4096).bfloat16()
    w = torch.randn(4096, 4096).bfloat16()
    torch.nn.functional.linear(a, w)
    t = time.perf_counter()
    torch.nn.functional.linear(a, w)
    gflops = 2 * 1448 * 4096 * 4096 / (time.perf_counter() - t) / 1e9
    layers = (4, 12) if gflops > 300 else (1, 2)
    log(f"[bench] cpu baseline: {threads} threads, bf16 GEMM {gflops:.0f} GFLOP/s, sample layers {layers}")
    gen = torch.Generator().manual_seed(SEED)
    medians, samples = [], {}
    for n_layers in layers:
        llm, drafter = build_models("cpu", torch.bfloat16, n_layers, SEED)
        cache = P.Cache(BATCH, PROMPT + NEW_TOKENS + WIDTH * LENGTH, n_layers, 32, 128, torch.bfloat16, "cpu")
        cache.data[:, :, :, :, :PROMPT] = torch.randn(cache.data[:, :, :, :, :PROMPT].shape, generator=gen).bfloat16()
        cache.set_length(PROMPT)
        ids = prompts("cpu")
        ctx = torch.randn(BATCH, 4096, generator=gen).bfloat16()
        tok = torch.randint(1, 32000, (BATCH,), generator=gen)
        with torch.inference_mode():
            step_times = []
            for i in range(1 + CPU_STEPS):  # the first pass pays one-time costs (allocator, kernel selection)
                cache.set_length(PROMPT)
                t = time.perf_counter()
                P.greedy_step(llm, drafter, ids, ctx, tok, cache, WIDTH, LENGTH, 0, tie="topk")
                if i > 0:
                    step_times.append(time.perf_counter() - t)
        samples[n_layers] = [round(x, 3) for x in step_times]
        medians.append(sorted(step_times)[len(step_times) // 2])
        log(f"[bench] cpu steps with {n_layers} layers: {samples[n_layers]} s")
        del llm, drafter, cache
    per_layer = (medians[1] - medians[0]) / (layers[1] - layers[0])
    full = medians[0] + (LLAMA_7B["num_hidden_layers"] - layers[0]) * per_layer
    return dict(
        value=round(per_seq_tokens * BATCH / full, 3), unit="tokens/s", cores=threads, kind="port",
        sample=(f"decode steps of the same workload (batch {BATCH}, context {PROMPT}, beam {WIDTH}x{LENGTH}, bf16; the "
                f"cache pre-filled, the prefill not timed) through the torch restatement with {layers[0]} and "
                f"{layers[1]} of 32 layers: median of {CPU_STEPS} steps each after one warm-up step "
                f"({medians[0]:.2f}s, {medians[1]:.2f}s), extrapolated linearly in the layer count to 32 layers = "
                f"{full:.2f}s/step; tokens per step taken from the GPU run"),
        seconds_per_step=round(full, 3),
        raw_step_seconds={str(k): v for k, v in samples.items()},
    )


def cpu_kernel_baselines(reps: int = 3):
    """Per-kernel CPU baselines: the torch restatement of each stage on the host cores, on the shapes
    of the kernel micro-benchmarks (kernel_bench.py).  Needs no GPU.  Prints one
    line per case: best of `reps` passes after one warm-up pass."""
    import numpy as np
    from oracle import torch_path as P
    from oracle import tree_oracle as T

    threads = torch.get_num_threads()
    log(f"[bench] per-kernel cpu baselines: {threads} threads, best of {reps} after one warm-up pass")
    rows = []

    def case(name, fn, n=reps):
        with torch.inference_mode():
            fn()
            best = float("inf")
            for _ in range(n):
                t = time.perf_counter()
                fn()
                best = min(best, time.perf_counter() - t)
        rows.append((name, best))
        print(f"{name:<78} cpu {best * 1e3:11.3f} ms   ({threads} threads)", flush=True)

    B, W, L, V, H, D = BATCH, WIDTH, LENGTH, 32000, 32, 128
    g = torch.Generator().manual_seed(SEED)
    beams = torch.from_numpy(T.synthetic_beams(B, W, L, seed=SEED))
    for prev in (0, 2548):
        pm = torch.ones(B, prev, dtype=torch.int64)
        case(f"tree_pack batch {B} prev {prev} (dedup, unpacker, pack, mask)", lambda: P.pack(beams, pm))

    # verification attention: additive bias + SDPA as the decoder layer issues them (one layer)
    rng = np.random.default_rng(SEED)
    for label, lens in (("cached length U[500,2548]", rng.integers(500, 2549, size=B)), ("cached length 525 for every row", np.full(B, 525))):
        S = int(lens.max())
        pm = torch.zeros(B, S, dtype=torch.int64)
        for b in range(B):
            pm[b, S - int(lens[b]):] = 1
        tok, _, mask, _ = P.pack(beams, pm)
        n = tok.shape[1]
        q = torch.randn(B, H, n, D, generator=g).bfloat16()
        k = torch.randn(B, H, S + n, D, generator=g).bfloat16()
        v = torch.randn(B, H, S + n, D, generator=g).bfloat16()

        def attn():
            m = P.rows_without_keys_to_true(mask)
            return torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=P.bias(m.unsqueeze(1), q.dtype))
        case(f"verify_attention {label} (n_q={n}, sum keys={int(lens.sum()) + B * n}), one layer", attn)

    # one beam-search step after the drafter's GEMMs: the chain of modeling_drafter.py:201-215
    logits = torch.randn(B, W, V, generator=g).bfloat16()
    log_p_beam = torch.randn(B, W, generator=g)

    def beam_step():
        x = logits - logits.max(dim=-1, keepdim=True).values
        x = P.top_k_filter(x)
        logp = torch.log_softmax(x, dim=-1)
        score = (logp + log_p_beam.unsqueeze(-1)).reshape(B, W * V)
        top, idx = torch.topk(score, W, dim=-1)
        return top, idx % V, idx // V
    case(f"beam_topk step, logits ({B},{W},{V}) bf16", beam_step)

    packed_logits = torch.randn(1448, V, generator=g).bfloat16()
    case("argmax packed bf16 logits (rows 1448)", lambda: packed_logits.argmax(dim=-1))
    case("verify_row_stats: top-50 filter + log_softmax of packed logits (rows 1448, fp32)",
         lambda: torch.log_softmax(P.top_k_filter(packed_logits.float()), dim=-1))
    hidden = torch.randn(B, 181, 4096, generator=g).bfloat16()
    unpacker = torch.randint(0, 181, (B, W, L), generator=g)
    case("unpack hidden (B,n,4096) bf16", lambda: P.unpack(hidden, unpacker))

    # KV cache: append of the tree rows' K (one layer), Cache.unpack and the re-alignment (32 layers)
    prev, n = 1500, 168
    cache = P.Cache(B, prev + n + 64, 32, H, D, torch.bfloat16, "cpu")
    cache.set_length(prev)
    new_k = torch.randn(B, H, n, D, generator=g).bfloat16()
    cos_t, sin_t = P._rope_tables(D, 10000.0, 2048, "cpu", torch.bfloat16)
    pos = torch.randint(prev, prev + L, (B, n), generator=g)

    def rope_append():
        cache.set_length(prev)
        c, s_ = cos_t[pos].unsqueeze(1), sin_t[pos].unsqueeze(1)
        cache.append(0, 0, P._rope(new_k, c, s_))
        cache.append(0, 1, new_k)
        cache.set_length(prev)
    case(f"rope + append prev {prev} n {n} (K rotated, V plain), one layer", rope_append)
    unp = torch.randint(0, n, (B, W, L), generator=g)

    def kv_unpack():
        cache.set_length(prev + n)
        cache.unpack(prev, unp)
        cache.set_length(prev)
    case(f"Cache.unpack prev {prev} n {n}, 32 layers", kv_unpack, n=2)
    ids = torch.randint(1, V, (B, prev), generator=g)
    n_tokens = torch.tensor([0, 1, 2, 3, 4, 4, 2, 1])[:B]
    seq_in_beam = torch.randint(0, W, (B,), generator=g)

    def realign():
        cache.set_length(prev + W * L)
        P.realign(ids, n_tokens, seq_in_beam, beams, cache, 0)
        cache.set_length(prev)
    case(f"realign ids + KV prev {prev}, accepted lengths differ, 32 layers", realign, n=2)
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--extra-steps", type=int, default=32,
                    help="timed steps of each additional operating point (long context, ragged acceptance); 0 skips them")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-kernels", action="store_true",
                    help="only time the CPU restatement of each stage on the micro-benchmark shapes (no GPU needed)")
    args = ap.parse_args()
    if args.cpu_kernels:
        cpu_kernel_baselines()
        return
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU (the decode step would shard by batch row with no "
            "exchange between the GPUs); --gpus must be 1")
        sys.exit(2)
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible; the HIP path has no CPU fallback")
        sys.exit(2)

    import recurrent_drafting_amd  # noqa: F401  (fails loudly if the HIP library is missing)

    run = gpu_run(args.steps, args.warmup, args.extra_steps)
    value = run["tokens"] / run["elapsed"]
    line = {
        "metric": "tokens/sec on 1 MI355X, Vicuna-7B-shape bs8 bw45 bl5 bf16; verify-step us",
        "value": round(value, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": run["steps"],
        "warmup": args.warmup,
        "ms_per_step": round(run["elapsed"] / run["steps"] * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic (seeded uniform prompts, random-init N(0,0.02) weights)",
        "config": {
            "workload": "end-to-end greedy decode step, Vicuna-7B-shaped Llama + ReDrafter head, "
                        "batch 8, prompt 500, beam 45x5, generation cap 2048",
            "context_tokens": list(run["context"]),
            "tokens_per_step_per_sequence": round(run["per_seq_tokens"], 3),
        },
        "verify_step_us": round(run["stage"]["verify_candidates"] * 1e6, 1),
        "stage_seconds_synchronised": {k: round(v, 6) for k, v in run["stage"].items()},
        "reference_style_tokens_per_second_per_sequence": round(run["ref_style_tokens_per_second"], 2),
        "roofline": attention_roofline(run),
        # the same decode step at other points of its operating range (the headline sits at the start
        # of the 500 -> 2548 trajectory, and random-init models accept no drafted token)
        "long_context": {k: summary_of(r) for k, r in run["others"].items() if k.startswith("context_")},
        "ragged_acceptance": {k: summary_of(r) for k, r in run["others"].items() if k.startswith("ragged_")},
        "ragged_prompts": {k: dict(summary_of(r), prompt_tokens=r["prompt_tokens"]) for k, r in run["others"].items()
                           if k.startswith("prompts_of_")},
        # speculative sampling (temperature 1): the headline's models and prompts, and the Llama-2-13B
        # shape at batch 16 with beam 64 x 5 (configuration 5 of the benchmark plan)
        "sampling": {k: sampling_summary(r) for k, r in run["others"].items() if "sampling" in k},
        # opt-in fused kernel against the default pair of kernels, same prompts, back to back (the
        # fused launch also rotates q and k and appends k and v: its time is not the attention's alone)
        "rope_attention_launches": {
            k[len("rope_attention_"):]: {"ms_per_step": round(r["elapsed"] / r["steps"] * 1e3, 3),
                                         "tokens_per_second": round(r["tokens"] / r["elapsed"], 2),
                                         "attn_mfma_kernel_avg_us": (lambda d: round(d[1] * 1e3 / d[0], 2) if d[0] else None)(
                                             r["dominant"].get("attn_mfma_kernel", (0, 0.0)))}
            for k, r in run["others"].items() if k.startswith("rope_attention_")},
        "kernel_avg_us": {k: round(ms * 1e3 / n, 2) for k, (n, ms) in sorted(run["kernels"].items())},
    }
    line["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline(run["per_seq_tokens"])
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
