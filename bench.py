#!/usr/bin/env python3
"""Throughput / latency benchmark of the BERT encoder path on one MI355X.

Protocol (the reference's: benchmark/turbo_benchmark_helper.py:29-34, benchmark_helper.py:17-61):
a random-init HuggingFace ``BertModel(BertConfig())`` (N(0,0.02) weights, pooler included) is
converted with ``turbo_transformers.BertModel.from_torch(model, device, "turbo")`` and run on
uniform random ids; W untimed warm-up forwards, then K timed ones.  A "step" is one forward of
the whole batch; sequences/s = batch / step time.

Headline workload: BERT-base fp16, batch 64 x seq 512 (the shape the MFMA/HBM targets are
stated on).  The same JSON line carries the other shapes of the metric (batch 1/20, seq 128,
the 20-request variable-length batch), the roofline of the dominant kernel measured live with
HIP events, and the CPU oracle timed on the host cores of the same box.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extras] [--no-cpu]
    python bench.py --only-extra smart_batch|albert_f16_b8_s256|base_int8_b20_s128   (one other configuration, for profiling)
    python bench.py --grid f16|bf16|f32   (the reference's fixed-length grid, this library beside PyTorch eager)
    python bench.py --yardstick           (what the box reaches outside this library: MFMA-only loop, hipBLASLt, copies)
"""
import argparse
import ctypes
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "f32": 157.3, "i8": 5000.0}
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (layers, hidden, heads, ffn, dtype, batch, seq)
    "base_f16_b64_s512": (12, 768, 12, 3072, "f16", 64, 512),
    "base_f16_b20_s128": (12, 768, 12, 3072, "f16", 20, 128),
    "base_f16_b1_s128": (12, 768, 12, 3072, "f16", 1, 128),
    "base_f32_b1_s128": (12, 768, 12, 3072, "f32", 1, 128),
    "base_f32_b64_s512": (12, 768, 12, 3072, "f32", 64, 512),
    "large_bf16_b64_s512": (24, 1024, 16, 4096, "bf16", 64, 512),
}
SMART_LENS_SEED = 0  # random.seed(0); randint(5, 500) x 20  (benchmark/benchmark_helper.py:77-79)


def forward_flops(layers, hidden, ffn, tokens, batch, seq):
    gemm = 2 * hidden * (3 * hidden + hidden + 2 * ffn) * tokens * layers
    attn = 4 * seq * hidden * tokens * layers
    return gemm, attn


def build_model(layers, hidden, heads, ffn, dtype):
    import torch
    from transformers import BertConfig, BertModel
    import turbo_transformers
    torch.manual_seed(1234)
    cfg = BertConfig(num_hidden_layers=layers, hidden_size=hidden, num_attention_heads=heads, intermediate_size=ffn)
    model = BertModel(cfg).eval()
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[dtype]
    model = model.to(tdt)
    dev = torch.device("cuda:0")
    return turbo_transformers.BertModel.from_torch(model, dev, "turbo"), model, cfg


def time_steps(fn, steps, warmup):
    """-> (mean ms per step, p50 ms, list of per-step ms); events on torch's current stream, which is
    the stream the kernels are enqueued on."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    events = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    events[0].record()
    for i in range(steps):
        fn()
        events[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    per = [events[i].elapsed_time(events[i + 1]) for i in range(steps)]
    total = events[0].elapsed_time(events[steps])
    per_sorted = sorted(per)
    return total / steps, per_sorted[len(per) // 2], per, wall_ms / steps


def run_dense(name, steps, warmup):
    import torch
    layers, hidden, heads, ffn, dtype, batch, seq = WORKLOADS[name]
    tmodel, hf_model, cfg = build_model(layers, hidden, heads, ffn, dtype)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, cfg.vocab_size - 1, (batch, seq), generator=g, dtype=torch.int64).cuda()
    ms, p50, _, wall = time_steps(lambda: tmodel(ids), steps, warmup)
    gemm, attn = forward_flops(layers, hidden, ffn, batch * seq, batch, seq)
    return {"workload": name, "dtype": dtype, "batch": batch, "seq": seq, "ms_per_step": ms, "p50_ms": p50,
            "host_wall_ms_per_step": wall, "seq_per_s": batch / ms * 1e3,
            "tflops": (gemm + attn) / ms / 1e9, "frac_of_mfma_peak": (gemm + attn) / ms / 1e9 / PEAK_TFLOPS[dtype]}


def run_grid(dtype, steps, warmup):
    """The reference's fixed-length grid (benchmark/run_gpu_fixed_benchmark.sh:20-22: batch 1 and 20, 10 ... 500 tokens,
    frameworks "turbo-transformers" and "torch"): ms per forward of this library and of the HuggingFace model run by
    PyTorch itself (eager, its default scaled-dot-product attention) on the same GPU, same weights, same ids."""
    import torch
    tmodel, hf_model, cfg = build_model(12, 768, 12, 3072, dtype)
    hf_model = hf_model.cuda()
    g = torch.Generator().manual_seed(0)
    rows = []
    shapes = [(batch, seq) for batch in (1, 20) for seq in (10, 20, 40, 60, 80, 100, 200, 300, 400, 500)]
    shapes.append((64, 512))  # not in the reference's grid: the shape the headline figure is quoted on
    for batch, seq in shapes:
        ids = torch.randint(0, cfg.vocab_size - 1, (batch, seq), generator=g, dtype=torch.int64).cuda()
        ms, _, _, _ = time_steps(lambda: tmodel(ids), steps, warmup)
        with torch.no_grad():
            ms_torch, _, _, _ = time_steps(lambda: hf_model(ids), steps, warmup)
        rows.append({"batch": batch, "seq": seq, "ms_per_step": ms, "pytorch_eager_ms_per_step": ms_torch,
                     "speedup": ms_torch / ms})
    return {"workload": "base_%s_fixed_length_grid" % dtype, "rows": rows}


def run_smart_batch(steps, warmup):
    """20 requests with lengths from the reference's recipe, packed (no padding) vs padded to the
    longest with a HuggingFace-style attention mask.  Two packed figures: the same 20 lengths every step (the
    per-batch device tables are then cached), and a fresh list of lengths every step, which is what a server
    sees (tables rebuilt and uploaded per batch, inside the timed region)."""
    import torch
    import turbo_transformers
    random.seed(SMART_LENS_SEED)
    lens = [random.randint(5, 500) for _ in range(20)]
    layers, hidden, heads, ffn = 12, 768, 12, 3072
    tmodel, hf_model, cfg = build_model(layers, hidden, heads, ffn, "f16")
    smart = turbo_transformers.BertModelSmartBatch.from_torch(hf_model, torch.device("cuda:0"))
    g = torch.Generator().manual_seed(0)
    inputs = [torch.randint(0, cfg.vocab_size - 1, (1, n), generator=g, dtype=torch.int64).cuda() for n in lens]
    ms_s, p50_s, _, _ = time_steps(lambda: smart(inputs, lens), steps, warmup)
    # fresh lengths: one batch per step, ids resident on the device before the clock starts
    batches = []
    for _ in range(steps + warmup):
        ls = [random.randint(5, 500) for _ in range(20)]
        batches.append((ls, [torch.randint(0, cfg.vocab_size - 1, (1, n), generator=g, dtype=torch.int64).cuda() for n in ls]))
    it = iter(batches)

    def fresh():
        ls, ins = next(it)
        smart(ins, ls)
    ms_f, p50_f, _, _ = time_steps(fresh, steps, warmup)
    tokens_f = sum(sum(ls) for ls, _ in batches[warmup:]) / steps
    max_len = max(lens)
    padded = torch.zeros(len(lens), max_len, dtype=torch.int64)
    mask = torch.zeros(len(lens), max_len, dtype=torch.int64)
    for i, t in enumerate(inputs):
        padded[i, :lens[i]] = t[0].cpu()
        mask[i, :lens[i]] = 1
    padded, mask = padded.cuda(), mask.cuda()
    ms_p, p50_p, _, _ = time_steps(lambda: tmodel(padded, attention_masks=mask), steps, warmup)
    return {"workload": "base_f16_smart_batch_20req", "lens_sum": sum(lens), "lens_max": max_len,
            "packed": {"ms_per_step": ms_s, "p50_ms": p50_s, "seq_per_s": len(lens) / ms_s * 1e3},
            "packed_fresh_lengths_each_step": {"ms_per_step": ms_f, "p50_ms": p50_f, "seq_per_s": 20 / ms_f * 1e3,
                                               "mean_tokens_per_step": tokens_f},
            "padded": {"ms_per_step": ms_p, "p50_ms": p50_p, "seq_per_s": len(lens) / ms_p * 1e3}}


# HBM-side traffic of one launch in bytes: a RECORDED constant, not something this run measures.  It comes from
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of `python3 bench.py --pmc-kernel <name>` (counter KiB
# scaled by what the calibration copy reads: x2.0 for FETCH_SIZE, x1.0 for WRITE_SIZE; summaries under profiles/).
# Keyed by (kernel of the roofline pass, dtype, batch, seq) AND by the kernel variant the library reports for that
# product (ttmi_gemm_describe): when the tile choice changes the record no longer applies and `traffic` is null.
MEASURED_TRAFFIC = {
    ("ffn1_gemm+bias+gelu", "f16", 64, 512): {"variant": "dma3_agpr4w_256x256", "fetch_bytes": 123162 * 2.0 * 1024,
                                              "write_bytes": 196608 * 1.0 * 1024},
}

COPY_ELEMS = 64 << 20  # fp32 elements of the calibration copy: reads 256 MiB, writes 256 MiB


def run_albert(steps, warmup):
    """ALBERT: embedding size 128 projected to 768, one shared layer applied 12 times; fp16, batch 8 x seq 256."""
    import torch
    import turbo_transformers
    from transformers import AlbertConfig, AlbertModel
    torch.manual_seed(1234)
    cfg = AlbertConfig(embedding_size=128, hidden_size=768, num_hidden_layers=12, num_attention_heads=12, intermediate_size=3072)
    model = AlbertModel(cfg).eval().half().cuda()
    tmodel = turbo_transformers.AlbertModel.from_torch(model)
    ids = torch.randint(0, cfg.vocab_size, (8, 256), generator=torch.Generator().manual_seed(0)).cuda()
    ms, p50, _, _ = time_steps(lambda: tmodel(ids), steps, warmup)
    return {"ms_per_step": ms, "p50_ms": p50, "seq_per_s": 8 / ms * 1e3}


def run_int8(steps, warmup):
    """BERT-base with every Linear as int8 x int8 -> int32 (dynamic per-tensor activation scale, per-channel weight
    scales), fp32 softmax / LayerNorm; batch 20 x seq 128."""
    import torch
    import turbo_transformers
    from transformers import BertConfig, BertModel
    torch.manual_seed(1234)
    cfg = BertConfig()
    model = BertModel(cfg).eval().cuda()
    qmodel = turbo_transformers.QBertModel.from_torch(model, backend="turbo")
    ids = torch.randint(0, cfg.vocab_size, (20, 128), generator=torch.Generator().manual_seed(0)).cuda()
    ms, p50, _, _ = time_steps(lambda: qmodel(ids), steps, warmup)
    return {"ms_per_step": ms, "p50_ms": p50, "seq_per_s": 20 / ms * 1e3}


def kernel_rooflines(dtype="f16", batch=64, seq=512, hidden=768, heads=12, ffn=3072, iters=20, only=None):
    """Each kernel of the layer alone, at its real shape, timed with HIP events on the work stream
    through the C ABI.  GEMMs: algorithmic FLOPs = 2*M*N*K against the MFMA peak; memory-bound
    kernels: algorithmic bytes (each tensor read / written once) against 8 TB/s."""
    import torch
    from turbotransformers_amd import capi
    lib = capi.load()
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[dtype]
    cdt = {"f16": capi.F16, "bf16": capi.BF16, "f32": capi.F32}[dtype]
    esz = 2 if dtype != "f32" else 4
    T, H, F, d = batch * seq, hidden, ffn, hidden // heads
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    S = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rnd = lambda *shape: (torch.randn(*shape, device="cuda") * 0.5).to(tdt)

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e3  # us

    # operand statistics as in the forward (LayerNorm-scale activations, N(0,0.02) weights): the MFMA
    # clock under load depends on how many operand bits toggle
    wgt = lambda *shape: (torch.randn(*shape, device="cuda") * 0.02).to(tdt)
    x, w_qkv, w_o, w_1, w_2 = rnd(T, H) * 2, wgt(3 * H, H), wgt(H, H), wgt(F, H), wgt(H, F)
    # biases 0, LayerNorm gamma 1 / beta 0: the values of a freshly initialised BertModel, as in the headline forward
    zeros = lambda n: torch.zeros(n, device="cuda", dtype=tdt)
    b_qkv, b_h, b_f, gam = zeros(3 * H), zeros(H), zeros(F), torch.ones(H, device="cuda", dtype=tdt)
    q, k, v = (rnd(batch, heads, seq, d) for _ in range(3))
    score = torch.empty(batch, heads, seq, seq, device="cuda", dtype=tdt)
    ctx, out, inter = rnd(T, H), torch.empty(T, H, device="cuda", dtype=tdt), rnd(T, F)
    mask = torch.zeros(batch, seq, device="cuda")

    def fused(a, w, c, m, n, kk, epi, **kw):
        args = capi.EpilogueArgs()
        for key, val in kw.items():
            setattr(args, key, val.data_ptr() if isinstance(val, torch.Tensor) else val)
        return lambda: capi.check(lib.ttmi_gemm_fused(P(a), P(w), P(c) if c is not None else None, m, n, kk, kk, kk, n, epi,
                                                      ctypes.byref(args), cdt, S()))

    if only is not None:
        # Counter runs (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE): one copy of known size through
        # ttmi_convert (fp32 -> fp32) to calibrate the counters' unit, then `iters` launches of the one kernel.
        src = torch.zeros(COPY_ELEMS, device="cuda")
        dst = torch.empty_like(src)
        capi.check(lib.ttmi_convert(P(src), capi.F32, P(dst), capi.F32, COPY_ELEMS, S()))
        torch.cuda.synchronize()
    res = {}
    gemms = {
        "qkv_gemm+bias+split": (fused(x, w_qkv, None, T, 3 * H, H, capi.EPI_QKV_SPLIT, bias=b_qkv, q=q, k=k, v=v, seq=seq,
                                      heads=heads, head_dim=d, v_seq_pitch=seq), 2 * T * 3 * H * H),
        "attn_out_gemm": (lambda: capi.check(lib.ttmi_gemm(P(ctx), P(w_o), P(out), T, H, H, H, H, H, 1, 1.0, 0.0, cdt, S())),
                          2 * T * H * H),
        "ffn1_gemm+bias+gelu": (fused(x, w_1, inter, T, F, H, capi.EPI_BIAS_ACT, bias=b_f, act=capi.ACT_GELU), 2 * T * F * H),
        "ffn2_gemm": (lambda: capi.check(lib.ttmi_gemm(P(inter), P(w_2), P(out), T, H, F, F, F, H, 1, 1.0, 0.0, cdt, S())),
                      2 * T * H * F),
        "qk_batched_gemm": (lambda: capi.check(lib.ttmi_gemm_strided_batched(
            P(q), P(k), P(score), seq, seq, d, d, d, seq, seq * d, seq * d, seq * seq, batch * heads, 1, 0.125, 0.0, cdt, S())),
            2 * T * seq * H),
        "pv_batched_gemm+merge": (lambda: capi.check(lib.ttmi_gemm_batched_heads(
            P(score), P(v), P(ctx), seq, d, seq, seq, d, H, heads, heads * seq * seq, seq * seq, heads * seq * d, seq * d,
            seq * H, d, batch, 0, 1.0, 0.0, cdt, S())), 2 * T * seq * H),
    }
    vt = torch.empty(batch, heads, d, seq, device="cuda", dtype=tdt).normal_()  # V kept transposed, as the layers do
    gemms["fused_attention"] = (lambda: capi.check(lib.ttmi_fused_attention(
        P(q), P(k), P(vt), P(mask), P(ctx), None, batch, heads, seq, d, seq, 0.125, cdt, S())), 4 * T * seq * H)
    if only is not None:
        membound_fns = {
            "add_bias_layer_norm": lambda: capi.check(lib.ttmi_add_bias_layer_norm(
                P(out), P(x), P(b_h), P(gam), P(b_h), T, H, 1e-12, cdt, S())),
        }
        fn = gemms[only][0] if only in gemms else membound_fns[only]
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        return None
    score.normal_()
    membound = {
        "apply_mask_and_softmax": (lambda: capi.check(lib.ttmi_apply_mask_and_softmax(
            P(score), P(mask), batch, heads, seq, seq, 1, 1.0, cdt, S())), 2 * batch * heads * seq * seq * esz + batch * seq * 4),
        "add_bias_layer_norm": (lambda: capi.check(lib.ttmi_add_bias_layer_norm(
            P(out), P(x), P(b_h), P(gam), P(b_h), T, H, 1e-12, cdt, S())), 3 * T * H * esz),
        "add_bias_gelu": (lambda: capi.check(lib.ttmi_add_bias_act(P(inter), P(b_f), T, F, capi.ACT_GELU, cdt, S())),
                          2 * T * F * esz),
    }
    # The kernels the forward launches are timed IN LAYER ORDER (QKV, attention, out-proj, LN, FFN1, FFN2, LN) and
    # by leave-one-out: duration(X) = time(layer sequence) - time(sequence without X), events only around whole
    # loops.  A kernel's clock and cache state depend on what ran before it (a GEMM repeated back to back runs
    # ~10 % slower than the same GEMM behind a memory-bound LayerNorm), and an event between two kernels makes
    # the second wait for the first to drain, which the forward does not do.
    layer_order = ["qkv_gemm+bias+split", "fused_attention", "attn_out_gemm", "add_bias_layer_norm",
                   "ffn1_gemm+bias+gelu", "ffn2_gemm", "add_bias_layer_norm"]
    fns = {name: gemms[name][0] for name in layer_order if name in gemms}
    fns["add_bias_layer_norm"] = membound["add_bias_layer_norm"][0]

    def time_sequence(names):
        for _ in range(2):
            for name in names:
                fns[name]()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            for name in names:
                fns[name]()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e3  # us per pass

    time_sequence(layer_order)  # first pass of the process: clocks and caches still settling
    # three rounds of (whole sequence, sequence without each kernel), median of the differences: one round's
    # difference of two ~0.7 ms figures carries a few microseconds of noise, which matters for the short kernels
    samples = {name: [] for name in dict.fromkeys(layer_order)}
    for _ in range(3):
        full = time_sequence(layer_order)
        if os.environ.get("TTMI_BENCH_DEBUG"):
            print("layer sequence: %.1f us" % full, file=sys.stderr)
        for name in samples:
            rest = [n for n in layer_order if n != name]
            without = time_sequence(rest)
            if os.environ.get("TTMI_BENCH_DEBUG"):
                print("  without %s: %.1f us" % (name, without), file=sys.stderr)
            samples[name].append((full - without) / layer_order.count(name))
    in_layer = {name: sorted(v)[len(v) // 2] for name, v in samples.items()}

    def variant(m, n, kk, epi, **kw):
        args = capi.EpilogueArgs()
        for key, val in kw.items():
            setattr(args, key, val)
        buf = ctypes.create_string_buffer(64)
        capi.check(lib.ttmi_gemm_describe(m, n, kk, epi, ctypes.byref(args), cdt, buf, 64))
        return buf.value.decode()
    variants = {"qkv_gemm+bias+split": variant(T, 3 * H, H, capi.EPI_QKV_SPLIT, seq=seq, heads=heads, head_dim=d, v_seq_pitch=seq),
                "attn_out_gemm": variant(T, H, H, capi.EPI_NONE), "ffn2_gemm": variant(T, H, F, capi.EPI_NONE),
                "ffn1_gemm+bias+gelu": variant(T, F, H, capi.EPI_BIAS_ACT, act=capi.ACT_GELU)}
    for name, (fn, flops) in gemms.items():
        us = in_layer[name] if name in in_layer else timed(fn)
        res[name] = {"bound": "mfma", "us": us, "achieved": flops / us / 1e6, "peak": PEAK_TFLOPS[dtype], "unit": "TFLOP/s",
                     "frac": flops / us / 1e6 / PEAK_TFLOPS[dtype], "flops_per_launch": flops, "variant": variants.get(name)}
    # AddBiasLayerNorm against the HBM roof: stand-alone over a ring of operand sets larger than the 256 MB
    # memory-side cache (each launch touches 100 MB that were last touched eight launches, 800 MB, ago), so that every
    # byte really comes from and goes to HBM.  Inside the layer its operands were written by the GEMM just before and
    # are partly served by that cache: the leave-one-out figure is kept as `in_layer_us`, but is no statement about HBM.
    ring = [(torch.empty(T, H, device="cuda", dtype=tdt).normal_(), torch.empty(T, H, device="cuda", dtype=tdt).normal_())
            for _ in range(8)]
    turn = [0]

    def cold_layer_norm():
        o, r = ring[turn[0] % len(ring)]
        turn[0] += 1
        capi.check(lib.ttmi_add_bias_layer_norm(P(o), P(r), P(b_h), P(gam), P(b_h), T, H, 1e-12, cdt, S()))
    cold_us = timed(cold_layer_norm)
    del ring
    for name, (fn, nbytes) in membound.items():
        us = in_layer[name] if name in in_layer else timed(fn)
        if name == "add_bias_layer_norm":
            res[name] = {"bound": "hbm", "us": cold_us, "in_layer_us": round(us, 1), "achieved": nbytes / cold_us / 1e3,
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": nbytes / cold_us / 1e3 / PEAK_HBM_GBS,
                         "bytes_per_launch": nbytes}
            continue
        res[name] = {"bound": "hbm", "us": us, "achieved": nbytes / us / 1e3, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": nbytes / us / 1e3 / PEAK_HBM_GBS, "bytes_per_launch": nbytes}
    # the layer classes use the fused attention kernel and the GEMM epilogues; the stand-alone forms
    # are measured for the kernel table but are not launched by the headline forward
    launches = {"qkv_gemm+bias+split": 1, "fused_attention": 1, "attn_out_gemm": 1, "ffn1_gemm+bias+gelu": 1,
                "ffn2_gemm": 1, "add_bias_layer_norm": 2}
    for name, r in res.items():
        r["launches_per_layer"] = launches.get(name, 0)
    return res


def run_yardstick(iters=20):
    """What this box reaches with code that is not this library's: the roofs the encoder kernels can be held against
    besides the published peaks.  Test-time only; nothing here is on a product path.  Prints a markdown report:
      (a) a loop of nothing but matrix instructions on register operands (ttmi_yardstick_mfma), both instruction
          shapes, zeros / N(0,1) / N(0,0.02^2) operands, with the shader clock the chip held (read inside the kernel);
      (b) ttmi_gemm / ttmi_gemm_fused(bias) against torch.nn.functional.linear (hipBLASLt) on the four encoder
          products of BERT-base and the two FFN products of BERT-large at 64 x 512 tokens, fp16 and bf16, same
          operands (activations N(0,1), weights N(0,0.02^2)), loops of `iters` launches;
      (c) the device copy rate: ttmi_convert fp32 -> fp32 (this library's copy kernel) and torch's copy_, 256 MiB and
          1 GiB per direction.
    Methodology as the reference's own GEMM micro-benchmark (benchmark/turbo_transformers/layers/kernels/
    matmul_benchmark.cpp:60-70: warm-up, a timed loop, 2*m*n*k FLOP per launch)."""
    import torch
    from turbotransformers_amd import capi
    lib = capi.load()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    S = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def timed(fn, n=iters):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e3  # us

    import turbo_transformers
    info = turbo_transformers.cxx.device_info()
    cus = int(info.get("compute_units", 256))
    out = ["# Yardsticks of this box (`python3 bench.py --yardstick`)", "",
           "Device: %s, %d compute units.  Test-time measurements; nothing here is on a product path." % (info["name"], cus), ""]

    # (a) matrix instructions only
    out += ["## (a) A loop of nothing but matrix instructions (register operands, eight wavefronts per CU)", "",
            "| type | instruction | operands | TFLOP/s | of 2.5 PFLOP/s | shader clock held (GHz) | matrix-pipe occupancy |",
            "|---|---|---|---|---|---|---|"]
    sink = torch.zeros(1, device="cuda")
    clocks = torch.zeros(2 * cus, dtype=torch.int64, device="cuda")
    loop_iters = 150000
    gen = torch.Generator(device="cuda").manual_seed(1)
    for dtype, tdt, cdt in (("f16", torch.float16, capi.F16), ("bf16", torch.bfloat16, capi.BF16)):
        pools = {"zeros": torch.zeros(65536, device="cuda", dtype=tdt),
                 "N(0,1)": torch.randn(65536, device="cuda", generator=gen).to(tdt),
                 "N(0,0.02^2)": (torch.randn(65536, device="cuda", generator=gen) * 0.02).to(tdt)}
        for block in (16, 32):
            for label, pool in pools.items():
                fn = lambda: capi.check(lib.ttmi_yardstick_mfma(block, cdt, P(pool), loop_iters, cus, P(sink), P(clocks), S()))
                fn()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                fn()
                e1.record()
                torch.cuda.synchronize()
                ms = e0.elapsed_time(e1)
                ck = clocks.view(cus, 2).double().cpu()
                if os.environ.get("TTMI_BENCH_DEBUG"):
                    print("yardstick %s %d %s: %.2f ms, shader cycles mean %.3e min %.3e max %.3e, 100 MHz ticks mean %.3e" % (
                        dtype, block, label, ms, ck[:, 0].mean(), ck[:, 0].min(), ck[:, 0].max(), ck[:, 1].mean()), file=sys.stderr)
                ghz = float((ck[:, 0] / ck[:, 1]).mean()) * 0.1  # shader cycles per tick of the 100 MHz clock
                flop = cus * 8 * loop_iters * 262144.0
                # share of the matrix pipes' cycles at the clock held: a SIMD retires 1024 FLOP per cycle in these types.
                # (The two counters are read by the first wavefront of each workgroup, which a SIMD serves ahead of its
                # younger neighbour: their ratio is the clock, but the time is taken from the events around the launch.)
                occupancy = flop / (ms * 1e-3) / (cus * 4 * 1024.0 * ghz * 1e9)
                out.append("| %s | %s | %s | %.0f | %.2f | %.2f | %.0f %% |" % (
                    dtype, "16x16x32" if block == 16 else "32x32x16", label, flop / ms / 1e9, flop / ms / 1e9 / 2500.0, ghz,
                    100 * occupancy))
    out.append("")

    # (b) this library's GEMM beside hipBLASLt
    out += ["## (b) `ttmi_gemm` beside `torch.nn.functional.linear` (hipBLASLt), 32768 rows, loops of %d launches" % iters, "",
            "Activations N(0,1), weights N(0,0.02^2), the same tensors for both; us per launch (TFLOP/s, share of 2.5 PFLOP/s).", "",
            "| product | N x K | type | form | this library | hipBLASLt | this / hipBLASLt time |", "|---|---|---|---|---|---|---|"]
    M = 64 * 512
    shapes = [("base QKV", 2304, 768), ("base out-proj", 768, 768), ("base FFN1", 3072, 768), ("base FFN2", 768, 3072),
              ("large FFN1", 4096, 1024), ("large FFN2", 1024, 4096)]
    for name, N, K in shapes:
        for dtype, tdt, cdt in (("f16", torch.float16, capi.F16), ("bf16", torch.bfloat16, capi.BF16)):
            A = torch.randn(M, K, device="cuda", generator=gen).to(tdt)
            W = (torch.randn(N, K, device="cuda", generator=gen) * 0.02).to(tdt)
            bias = (torch.randn(N, device="cuda", generator=gen) * 0.02).to(tdt)
            C = torch.empty(M, N, device="cuda", dtype=tdt)
            args = capi.EpilogueArgs()
            args.bias = bias.data_ptr()
            forms = {"bare": (lambda: capi.check(lib.ttmi_gemm(P(A), P(W), P(C), M, N, K, K, K, N, 1, 1.0, 0.0, cdt, S())),
                              lambda: torch.nn.functional.linear(A, W)),
                     "+ bias": (lambda: capi.check(lib.ttmi_gemm_fused(P(A), P(W), P(C), M, N, K, K, K, N, capi.EPI_BIAS,
                                                                       ctypes.byref(args), cdt, S())),
                                lambda: torch.nn.functional.linear(A, W, bias))}
            flop = 2.0 * M * N * K
            for form, (mine, theirs) in forms.items():
                us_m, us_t = timed(mine), timed(theirs)
                out.append("| %s | %d x %d | %s | %s | %.1f (%.0f, %.2f) | %.1f (%.0f, %.2f) | %.2f |" % (
                    name, N, K, dtype, form, us_m, flop / us_m / 1e6, flop / us_m / 1e6 / 2500.0, us_t, flop / us_t / 1e6,
                    flop / us_t / 1e6 / 2500.0, us_m / us_t))
            del A, W, C
    out.append("")

    # (c) copies
    out += ["## (c) Device copy rate (bytes read + bytes written, over the time of a launch)", "",
            "| copy | bytes each way | us | GB/s | of 8 TB/s |", "|---|---|---|---|---|"]
    for mib in (256, 1024):
        n = mib << 18  # fp32 elements
        src = torch.randn(n, device="cuda")
        dst = torch.empty_like(src)
        for label, fn in (("ttmi_convert fp32 -> fp32", lambda: capi.check(lib.ttmi_convert(P(src), capi.F32, P(dst), capi.F32, n, S()))),
                          ("torch copy_", lambda: dst.copy_(src))):
            us = timed(fn)
            gbs = 2.0 * n * 4 / us / 1e3
            out.append("| %s | %d MiB | %.1f | %.0f | %.2f |" % (label, mib, us, gbs, gbs / PEAK_HBM_GBS))
        del src, dst
    print("\n".join(out))


def run_ffn2_probe(iters=20, batch=64, seq=512, hidden=768, ffn=3072):
    """Why the second FFN product (32768 x 768 x 3072, fp16) takes longer inside the forward than in a loop of itself:
    loops of short kernel sequences through the C ABI, timed with events around the whole loop (us per pass).  The
    interaction cost of a pair is t(pair) - t(first alone) - t(second alone).  `own` = FFN2 reads what the FFN1 launch
    in front of it has just written (201 MB); `other` = it reads a second buffer of the same statistics that nothing
    writes, so that only clocks and caches, not the data dependency, tie the two launches together."""
    import torch
    from turbotransformers_amd import capi
    lib = capi.load()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    S = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    T, H, F = batch * seq, hidden, ffn
    tdt, cdt = torch.float16, capi.F16
    x = torch.randn(T, H, device="cuda").to(tdt)
    w1, w2 = (torch.randn(F, H, device="cuda") * 0.02).to(tdt), (torch.randn(H, F, device="cuda") * 0.02).to(tdt)
    b1, bh, gam = torch.zeros(F, device="cuda", dtype=tdt), torch.zeros(H, device="cuda", dtype=tdt), torch.ones(H, device="cuda", dtype=tdt)
    own = torch.empty(T, F, device="cuda", dtype=tdt)
    out, res = torch.empty(T, H, device="cuda", dtype=tdt), torch.randn(T, H, device="cuda").to(tdt)
    args = capi.EpilogueArgs()
    args.bias, args.act = b1.data_ptr(), capi.ACT_GELU
    ffn1 = lambda: capi.check(lib.ttmi_gemm_fused(P(x), P(w1), P(own), T, F, H, H, H, F, capi.EPI_BIAS_ACT, ctypes.byref(args), cdt, S()))
    ffn1()
    other = own.clone()
    args_b = capi.EpilogueArgs()
    args_b.bias = b1.data_ptr()
    ffn1_b = lambda: capi.check(lib.ttmi_gemm_fused(P(x), P(w1), P(own), T, F, H, H, H, F, capi.EPI_BIAS, ctypes.byref(args_b), cdt, S()))
    ffn2 = lambda a: (lambda: capi.check(lib.ttmi_gemm(P(a), P(w2), P(out), T, H, F, F, F, H, 1, 1.0, 0.0, cdt, S())))
    ln = lambda: capi.check(lib.ttmi_add_bias_layer_norm(P(out), P(res), P(bh), P(gam), P(bh), T, H, 1e-12, cdt, S()))
    copy_src, copy_dst = torch.randn(64 << 20, device="cuda"), torch.empty(64 << 20, device="cuda")
    flush = lambda: capi.check(lib.ttmi_convert(P(copy_src), capi.F32, P(copy_dst), capi.F32, 64 << 20, S()))  # 512 MB through the caches

    def timed(fns):
        for _ in range(3):
            for fn in fns:
                fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            for fn in fns:
                fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e3

    cases = [("FFN2 (other)", [ffn2(other)]), ("FFN1", [ffn1]), ("LayerNorm", [ln]), ("copy 2 x 256 MiB", [flush]),
             ("FFN1, FFN2 (own)", [ffn1, ffn2(own)]), ("FFN1, FFN2 (other)", [ffn1, ffn2(other)]),
             ("LayerNorm, FFN2 (other)", [ln, ffn2(other)]), ("copy, FFN2 (other)", [flush, ffn2(other)]),
             ("LayerNorm, FFN1, FFN2 (own), LayerNorm", [ln, ffn1, ffn2(own), ln]),
             ("FFN2 (other), FFN2 (other)", [ffn2(other), ffn2(other)]),
             # what the GELU in FFN1's epilogue costs in layer order: the same sequence with a bias-only epilogue
             ("FFN1 bias only", [ffn1_b]),
             ("LayerNorm, FFN1 bias only, FFN2 (own), LayerNorm", [ln, ffn1_b, ffn2(own), ln])]
    t = {}
    out_lines = ["# The second FFN product inside the forward and alone (`python3 bench.py --ffn2-probe`)", "",
                 "fp16, %d x %d tokens; loops of %d passes of each sequence, us per pass (events around the whole loop)." % (batch, seq, iters), "",
                 "| sequence | us per pass | sum of its parts alone | interaction |", "|---|---|---|---|"]
    for rnd in range(2):  # two rounds, the second is reported: clocks and caches settled
        for name, fns in cases:
            t[name] = timed(fns)
    single = {"FFN2 (own)": t["FFN2 (other)"], "FFN2 (other)": t["FFN2 (other)"], "FFN1": t["FFN1"], "LayerNorm": t["LayerNorm"],
              "copy": t["copy 2 x 256 MiB"], "FFN1 bias only": t["FFN1 bias only"]}
    for name, _ in cases:
        parts = [p.strip() for p in name.split(",")]
        if len(parts) == 1:
            out_lines.append("| %s | %.1f | | |" % (name, t[name]))
        else:
            alone = sum(single[p] for p in parts)
            out_lines.append("| %s | %.1f | %.1f | %+.1f |" % (name, t[name], alone, t[name] - alone))
    out_lines += ["", "GELU in FFN1's epilogue: %.1f us alone in a loop, %.1f us in layer order." % (
        t["FFN1"] - t["FFN1 bias only"],
        t["LayerNorm, FFN1, FFN2 (own), LayerNorm"] - t["LayerNorm, FFN1 bias only, FFN2 (own), LayerNorm"])]
    print("\n".join(out_lines))


def run_pmc_gemm(spec):
    """Counter-collection helper: one bare product, `which,M,N,K,dtype` with which = ttmi (this library's ttmi_gemm) or
    blaslt (torch.nn.functional.linear = hipBLASLt), on N(0,1) activations and N(0,0.02^2) weights; three warm-up and ten
    timed launches, one line of text.  Run under `rocprofv3 --pmc ...` it puts the same counters on both kernels."""
    import torch
    from turbotransformers_amd import capi
    which, m, n, k, dt = spec.split(",")
    m, n, k = int(m), int(n), int(k)
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16}[dt]
    cdt = {"f16": capi.F16, "bf16": capi.BF16}[dt]
    torch.manual_seed(0)
    a = torch.randn(m, k, device="cuda").to(tdt)
    w = (torch.randn(n, k, device="cuda") * 0.02).to(tdt)
    out = torch.empty(m, n, device="cuda", dtype=tdt)
    if which == "ttmi":
        lib = capi.load()
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        fn = lambda: capi.check(lib.ttmi_gemm(P(a), P(w), P(out), m, n, k, k, k, n, 1, 1.0, 0.0, cdt,
                                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    else:
        fn = lambda: torch.nn.functional.linear(a, w)
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        fn()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / 10 * 1e3
    print("%s %d x %d x %d %s: %.1f us per launch, %.0f TFLOP/s" % (which, m, n, k, dt, us, 2.0 * m * n * k / us / 1e6))


def cpu_baseline(seqs=4, seq=512, repeats=2):
    """The CPU oracle (an in-repo restatement of the reference's CPU branch: OpenMP loops + cblas_sgemm)
    on a bounded sample of the headline workload: `seqs` of the 64 sequences, all 12 layers, fp32; timed with 4 and
    8 threads (benchmark/run_cpu_fixed_benchmark.sh:16 of the reference) and with every core the process may use,
    which is the headline `value`."""
    import numpy as np
    from oracle.loader import Oracle
    o = Oracle()
    threads = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    rng = np.random.default_rng(1234)
    H, F, heads, L = 768, 3072, 12, 12
    n = lambda *s: (rng.standard_normal(s, np.float32) * 0.02)
    layers = [{"qkv_w": n(H, 3 * H), "qkv_b": np.zeros(3 * H, np.float32), "attn_out_w": n(H, H),
               "attn_out_b": np.zeros(H, np.float32), "attn_ln_g": np.ones(H, np.float32), "attn_ln_b": np.zeros(H, np.float32),
               "inter_w": n(H, F), "inter_b": np.zeros(F, np.float32), "out_w": n(F, H), "out_b": np.zeros(H, np.float32),
               "out_ln_g": np.ones(H, np.float32), "out_ln_b": np.zeros(H, np.float32)} for _ in range(L)]
    x = rng.standard_normal((seqs, seq, H), np.float32)
    mask = np.zeros((seqs, 1, 1, seq), np.float32)
    x1, m1 = x[:1, :128].copy(), mask[:1, :, :, :128].copy()
    by_threads = {}
    for t in sorted({t for t in (4, 8, threads) if t <= threads}):
        o.set_num_threads(t)
        o.bert_encoder(x[:1, :64].copy(), mask[:1, :, :, :64].copy(), layers, heads)  # warm-up (thread pools, BLAS init)
        reps = repeats if t == threads else 1
        t0 = time.perf_counter()
        for _ in range(reps):
            o.bert_encoder(x, mask, layers, heads)
        dt = (time.perf_counter() - t0) / reps
        # the reference's own CPU-runnable case (batch 1 x seq 128, fp32), median of 8 forwards
        small = []
        for _ in range(8):
            t1 = time.perf_counter()
            o.bert_encoder(x1, m1, layers, heads)
            small.append(time.perf_counter() - t1)
        by_threads[t] = {"seq_per_s": seqs / dt, "seconds_per_forward": dt, "b1_s128_ms_per_forward": sorted(small)[len(small) // 2] * 1e3}
    top = by_threads[threads]
    return {"value": top["seq_per_s"], "b1_s128_ms_per_forward": top["b1_s128_ms_per_forward"], "unit": "seq/s", "cores": threads,
            "kind": "port",
            "sample": "%d of the 64 sequences (batch %d x seq %d), 12 encoder layers, fp32, %d timed forwards after a warm-up; "
                      "BLAS: %s" % (seqs, seqs, seq, repeats, os.path.basename(o.blas_name())),
            "seconds_per_forward": top["seconds_per_forward"],
            "by_threads": {str(t): {k: round(v, 4) for k, v in r.items()} for t, r in by_threads.items()}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="base_f16_b64_s512", choices=sorted(WORKLOADS))
    ap.add_argument("--no-extras", action="store_true", help="skip the other shapes of the metric")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel roofline pass")
    ap.add_argument("--only-extra", default=None, choices=["smart_batch", "albert_f16_b8_s256", "base_int8_b20_s128"],
                    help="profiling helper: run just this other configuration of the metric, print its figures, exit")
    ap.add_argument("--grid", default=None, choices=["f16", "bf16", "f32"],
                    help="time the reference's fixed-length grid (batch 1/20 x 10..500 tokens) beside PyTorch eager, print it as JSON and exit")
    ap.add_argument("--yardstick", action="store_true",
                    help="print what this box reaches outside this library (a loop of matrix instructions, hipBLASLt on "
                         "the encoder's products, copy rates) as a markdown report and exit")
    ap.add_argument("--ffn2-probe", action="store_true",
                    help="time the second FFN product alone and behind the kernels that precede it in the forward "
                         "(markdown report), exit")
    ap.add_argument("--pmc-kernel", default=None,
                    help="counter-collection helper: run one calibration copy and a few launches of the named kernel "
                         "of the roofline pass (e.g. ffn1_gemm+bias+gelu), print nothing, exit")
    ap.add_argument("--pmc-gemm", default=None, metavar="WHICH,M,N,K,DTYPE",
                    help="counter-collection helper: a few launches of one bare product by this library (ttmi) or by "
                         "hipBLASLt (blaslt), e.g. ttmi,32768,1024,4096,bf16; prints its time, exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU (requests are independent; there is no multi-GPU step to time); "
                 "--gpus %d is not supported" % args.gpus)

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import turbo_transformers  # noqa: F401  (fails loudly if the native libraries are missing)

    layers, hidden, heads, ffn, dtype, batch, seq = WORKLOADS[args.workload]
    if args.pmc_kernel:
        kernel_rooflines(dtype, batch, seq, hidden, heads, ffn, iters=3, only=args.pmc_kernel)
        return
    if args.pmc_gemm:
        run_pmc_gemm(args.pmc_gemm)
        return
    if args.grid:
        print(json.dumps(run_grid(args.grid, args.steps, args.warmup)))
        return
    if args.yardstick:
        run_yardstick()
        return
    if args.ffn2_probe:
        run_ffn2_probe()
        return
    if args.only_extra:
        run = {"smart_batch": lambda: run_smart_batch(max(10, args.steps // 2), args.warmup),
               "albert_f16_b8_s256": lambda: run_albert(args.steps, args.warmup),
               "base_int8_b20_s128": lambda: run_int8(args.steps, args.warmup)}[args.only_extra]
        print(json.dumps({args.only_extra: run()}))
        return
    head = run_dense(args.workload, args.steps, args.warmup)
    line = {
        "metric": "bert_base_sequences_per_second", "value": head["seq_per_s"], "unit": "seq/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"], "p50_latency_ms": head["p50_ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": "%s: %d-layer BERT (hidden %d, %d heads, FFN %d, pooler) %s, batch %d x seq %d, random-init "
                               "N(0,0.02) weights, uniform random ids, via turbo_transformers.BertModel.from_torch"
                               % (args.workload, layers, hidden, heads, ffn, dtype, batch, seq)},
        "forward_tflops": head["tflops"], "forward_frac_of_mfma_peak": head["frac_of_mfma_peak"],
        "device": turbo_transformers.cxx.device_info()["name"],
    }
    if not args.no_kernels:
        kr = kernel_rooflines(dtype, batch, seq, hidden, heads, ffn)
        # dominant kernel = largest share of the layer time
        dom = max(kr, key=lambda k: kr[k].get("in_layer_us", kr[k]["us"]) * kr[k]["launches_per_layer"])
        r = kr[dom]
        line["roofline"] = {"kernel": dom, "bound": r["bound"], "achieved": r["achieved"], "peak": r["peak"], "unit": r["unit"],
                            "frac": r["frac"], "traffic": None, "avg_launch_us": r["us"]}
        t = MEASURED_TRAFFIC.get((dom, dtype, batch, seq))
        variant = kr[dom].get("variant")
        line["roofline"]["kernel_variant"] = variant
        if t is not None and t["variant"] == variant:
            line["roofline"]["traffic"] = t["fetch_bytes"] + t["write_bytes"]
            line["roofline"]["traffic_detail"] = dict(t, unit="bytes per launch", source="recorded rocprofv3 counter run "
                                                      "(profiles/ffn1_gemm_f16_b64_s512_traffic.md), not measured by this run",
                                                      algorithmic_bytes=2 * (batch * seq * hidden + hidden * ffn + batch * seq * ffn))
        line["kernel_rooflines"] = {k: {"bound": v["bound"], "us": round(v["us"], 1), "achieved": round(v["achieved"], 1),
                                        "unit": v["unit"], "frac": round(v["frac"], 4),
                                        "launches_per_layer": v["launches_per_layer"],
                                        **({"variant": v["variant"]} if v.get("variant") else {}),
                                        **({"in_layer_us": v["in_layer_us"]} if "in_layer_us" in v else {})}
                                    for k, v in kr.items()}
    else:
        line["roofline"] = None
    if not args.no_extras:
        extras = {}
        for name in ("base_f16_b1_s128", "base_f16_b20_s128", "base_f32_b1_s128"):
            if name != args.workload:
                r = run_dense(name, max(20, args.steps), args.warmup)
                extras[name] = {k: r[k] for k in ("ms_per_step", "p50_ms", "seq_per_s", "host_wall_ms_per_step")}
        extras["smart_batch"] = run_smart_batch(max(10, args.steps // 2), args.warmup)
        r = run_dense("large_bf16_b64_s512", 10, 2)
        extras["large_bf16_b64_s512"] = {k: r[k] for k in ("ms_per_step", "p50_ms", "seq_per_s", "tflops")}
        if args.workload != "base_f32_b64_s512":  # the reference's own element type at the headline shape
            r = run_dense("base_f32_b64_s512", 5, 2)
            extras["base_f32_b64_s512"] = {k: r[k] for k in ("ms_per_step", "p50_ms", "seq_per_s", "tflops", "frac_of_mfma_peak")}
        extras["albert_f16_b8_s256"] = run_albert(30, args.warmup)
        extras["base_int8_b20_s128"] = run_int8(30, args.warmup)
        line["other_workloads"] = extras
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline()
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
