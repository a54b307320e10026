#!/usr/bin/env python3
"""Benchmark of the int8 transformer-layer forward path on one MI355X.

Default workload (``--workload bert_base``): the BERT-base-shaped int8 encoder stack --
12 layers, hidden 768, 12 heads, FFN 3072 GELU, batch 32 x max seq 128, per-sequence
valid lengths uniform in [32, 128] with right padding, token ids uniform over a
30522 vocabulary, random-init weights ~N(0, 0.02) quantised per tensor -- run
through the drop-in entry point ``QuantBert(path, max_batch)`` / ``LSModel::Infer``.
A step is one ``Infer()`` over one batch whose token ids are already resident in
HBM.  ``value`` = batch * seq_len * steps / wall time of the timed steps (padded
tokens counted, as the reference's b32 x s128 figures do).

The JSON line also carries
  roofline       the dominant kernel launch (by total time) among the int8 GEMM sites
                 of a layer (one kernel instantiation at one shape), timed with HIP events
                 on the model's stream during a second, instrumented pass over the same
                 steps: achieved = 2*M*N*K per launch / mean launch time, against the
                 5.0 POP/s dense int8 MFMA peak;
  fused_kernels  the memory-bound fused kernels of one encoder layer at this workload's
                 shapes, each timed alone over back-to-back launches queued behind a long
                 kernel (so the host's launch cost is not what is measured): achieved
                 GB/s = algorithmic bytes (every operand touched once) / mean time per
                 launch, against the 8 TB/s HBM peak;
  gemm_microbench  the 4096x4096x1024 and 4096x1024x4096 int8 products (and 8192^3; uniform codes in
                 [-127, 127]) with int32 output, requantised int8 output and the fused
                 bias+GELU+requantisation epilogue, and the stand-alone
                 dequant-bias-GELU-requant kernel, timed the same way;
  cpu_baseline   the CPU oracle (a C port of the reference's algorithm, OpenMP) timed
                 on this host on a bounded sample of the same workload, and beside it
                 (``torch_cpu``) a PyTorch-CPU restatement of the layer with the formulas of
                 the reference's kernel tests (F.linear on dequantised codes, F.layer_norm,
                 tanh-GELU, fake quantisation between the stages) -- baselines only.

``step_ms`` holds the median, 10th and 90th percentile of the per-step times between HIP
events recorded on the model's stream; ``roofline.measured_peak`` is what a loop of nothing
but register-resident int8 MFMAs sustains on this box, ``frac_of_measured_peak`` the dominant
launch against that.

``--workload transformer_big`` and ``--workload gpt2_medium`` time the two generation
workloads (beam-search translation, greedy GPT generation) through ``QuantTransformer`` /
``QuantGpt`` in benchmark mode: generated tokens/s over whole ``Infer()`` calls, the time of a
decode step between HIP events on the model's stream, its launches, a roofline block (one step's
algorithmic HBM bytes -- weights, cached keys and values, logits -- against 8 TB/s) and the CPU
oracle on a few steps of the same width.  The default line carries both under ``generation``.
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_MFMA_PEAK_TOPS = 5000.0  # dense int8, MI355X
HBM_PEAK_GBS = 8000.0

BATCH, SEQ = 32, 128


def cpu_baseline(cfg, msg, ids, layers=12):
    """Oracle timed on the host: `layers` encoder layers of the real width at the full
    b32 x s128 batch, scaled to the 12-layer stack."""
    from oracle import oracle
    from oracle.model_io import oracle_weights_from_message
    sub = dict(cfg, n_layer=layers)
    sub_msg = dict(msg, encoder_stack=msg["encoder_stack"][:layers])
    w = oracle_weights_from_message(sub_msg, sub)
    oracle.quant_bert_encoder(w, ids[:2])  # page in, spin up the OpenMP team
    t0 = time.perf_counter()
    oracle.quant_bert_encoder(w, ids)
    dt = time.perf_counter() - t0
    full = dt * cfg["n_layer"] / layers
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return {"value": ids.size / full, "unit": "tokens/s", "cores": cores, "kind": "port",
            "what": "oracle/ls_oracle*.c: plain-C restatement of the reference's int8 kernels, OpenMP",
            "sample": "one step: %d of %d encoder layers at batch %d x seq %d, %.1f s of CPU work%s"
                      % (layers, cfg["n_layer"], ids.shape[0], ids.shape[1], dt,
                         "" if layers == cfg["n_layer"] else ", scaled to the full stack")}


def torch_cpu_baseline(cfg, ids, layers=2):
    """PyTorch-CPU restatement of the int8 encoder layer with the formulas the reference's
    kernel tests use as their baselines (tests/test_ls_kernels.py: F.layer_norm, F.linear on
    dequantised int8 codes, relu / gelu of the dequantised sum, quantise by
    clamp(floor(x / scale + 0.5))), fp32, all host threads.  A baseline, not a checker:
    `layers` layers at the full batch, scaled to the stack."""
    import torch
    import torch.nn.functional as F
    B, S = ids.shape
    H, I, h = cfg["hidden"], cfg["inner"], cfg["head_num"]
    d = H // h
    g = torch.Generator().manual_seed(0)

    def fq(x, clip):  # fake quantisation: quantise + dequantise
        s = clip / 127.0
        return torch.clamp(torch.floor(x / s + 0.5), -127, 127) * s

    ws = [dict(qkv=fq(torch.randn(3 * H, H, generator=g) * 0.02, 0.08), o=fq(torch.randn(H, H, generator=g) * 0.02, 0.08),
               f1=fq(torch.randn(I, H, generator=g) * 0.02, 0.08), f2=fq(torch.randn(H, I, generator=g) * 0.02, 0.08),
               b_qkv=torch.zeros(3 * H), b_o=torch.zeros(H), b1=torch.zeros(I), b2=torch.zeros(H),
               g1=torch.ones(H), be1=torch.zeros(H), g2=torch.ones(H), be2=torch.zeros(H)) for _ in range(layers)]
    x = torch.randn(B, S, H, generator=g)
    mask = torch.from_numpy((ids == cfg["padding_id"])).view(B, 1, 1, S)

    def layer(x, w):
        B = x.shape[0]
        mask_b = mask[:B]
        q0 = fq(F.layer_norm(x, (H,), w["g1"], w["be1"], 1e-12), 4.0)
        qkv = fq(F.linear(q0, w["qkv"]), 8.0) + w["b_qkv"]
        q, k, v = (t.reshape(B, S, h, d).transpose(1, 2) for t in qkv.split(H, dim=-1))
        p = torch.softmax((q @ k.transpose(-1, -2) / d ** 0.5).masked_fill(mask_b, -1e8), -1)
        ctx = fq((p @ v).transpose(1, 2).reshape(B, S, H), 2.0)
        r = fq(F.linear(ctx, w["o"]), 4.0) + w["b_o"] + x
        q1 = fq(F.layer_norm(r, (H,), w["g2"], w["be2"], 1e-12), 4.0)
        a = fq(F.gelu(fq(F.linear(q1, w["f1"]), 8.0) + w["b1"], approximate="tanh"), 6.0)
        return F.linear(a, w["f2"]) + w["b2"] + r

    with torch.no_grad():
        layer(x[:2], ws[0])
        t0 = time.perf_counter()
        for w in ws:
            x = layer(x, w)
        dt = time.perf_counter() - t0
    full = dt * cfg["n_layer"] / layers
    return {"value": ids.size / full, "unit": "tokens/s", "cores": torch.get_num_threads(),
            "kind": "PyTorch-CPU fp32 restatement of the reference's kernel-test baselines",
            "sample": "%d of %d layers at batch %d x seq %d, %.1f s of CPU work, scaled to the full stack"
                      % (layers, cfg["n_layer"], B, S, dt)}


def measured_mfma_peak(reps=5):
    """TOP/s of a loop of independent register-resident int8 MFMAs (lsh_mfma_i8_peak_probe),
    2 workgroups per compute unit, timed with HIP events on the launch stream."""
    import torch
    from lightseq_amd import kernels as K
    wgs = 2 * torch.cuda.get_device_properties(0).multi_processor_count
    out = torch.zeros(wgs * 256, dtype=torch.int32, device="cuda:0")
    K.mfma_i8_peak_probe(out, wgs, 200)
    torch.cuda.synchronize()
    best = 0.0
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        ops = K.mfma_i8_peak_probe(out, wgs, 4000)
        e1.record()
        torch.cuda.synchronize()
        best = max(best, ops / (e0.elapsed_time(e1) * 1e-3) / 1e12)
    return best


def fused_kernel_rates(cfg, reps=50, BATCH=BATCH):
    """Each memory-bound kernel of one encoder layer alone, at the workload's shapes (or, with
    another ``BATCH``, on tensors large enough that launch and first-byte costs vanish)."""
    import torch
    from lightseq_amd import kernels as K
    dev = "cuda:0"
    M, H, I, h = BATCH * SEQ, cfg["hidden"], cfg["inner"], cfg["head_num"]
    d = H // h
    g = torch.Generator(device=dev).manual_seed(0)

    def i8(*shape):
        return torch.randint(-127, 128, shape, dtype=torch.int8, device=dev, generator=g)

    def f16(*shape):
        return torch.randn(*shape, dtype=torch.float16, device=dev, generator=g)

    x16, res16 = f16(M, H), f16(M, H)
    q8_h, q8_3h, q8_i, out8_i = i8(M, H), i8(M, 3 * H), i8(M, I), i8(M, I)
    acc32 = torch.randint(-2 ** 20, 2 ** 20, (M, H), dtype=torch.int32, device=dev, generator=g)
    gam, bet, rb = f16(H), f16(H), f16(H)
    b3h, bi = f16(3 * H), f16(I)
    qkv = torch.zeros(3, BATCH, h, SEQ, d, dtype=torch.float16, device=dev)
    qkv.copy_(f16(3, BATCH, h, SEQ, d))
    mask = torch.zeros(BATCH, SEQ, dtype=torch.int32, device=dev)
    ctx8 = i8(M, H)
    mbd = M * H
    cases = [
        # name, algorithmic bytes, launcher
        ("launch_quantize_tensor f16->i8", M * H * 3,
         lambda: K.launch_quantize_tensor(x16, q8_h, M, H, 30.0)),
        ("launch_dequantize_tensor i32->f16", M * H * 6,
         lambda: K.launch_dequantize_tensor(acc32, x16, M, H, 1e-4)),
        ("ker_residual_bias_ln_i8I_i8O", M * H * (1 + 2 + 1 + 2),
         lambda: K.ker_residual_bias_ln_i8I_i8O_launcher(q8_h, gam, bet, rb, ctx8, res16, M, H,
                                                         0.05, 30.0, 1024, True)),
        ("ker_residual_bias_ln_i32I_i8O", M * H * (4 + 2 + 1 + 2),
         lambda: K.ker_residual_bias_ln_i32I_i8O_launcher(acc32, gam, bet, rb, ctx8, res16, M, H,
                                                          1e-4, 30.0, 1024, True)),
        ("ker_bias_gelu_i8I_i8O", M * I * 2,
         lambda: K.ker_bias_gelu_i8I_i8O_launcher(M, q8_i, out8_i, bi, I, 0.05, 30.0)),
        ("ker_arrange_encself_qkv_i8I", M * 3 * H * (1 + 2),
         lambda: K.ker_arrange_encself_qkv_i8I_launcher(M, H, q8_3h, b3h, qkv, mbd, SEQ, d, h, 1024,
                                                        0.05)),
        ("encself_attention (fused QK^T, softmax, PV, merge+quant)", M * H * (3 * 2 + 1),
         lambda: K.encself_attention(qkv[0], qkv[1], qkv[2], mask, None, ctx8, 30.0, BATCH, SEQ, h,
                                     d)),
        ("encself_attention on the int8 QKV product (what the model runs)", M * H * (3 + 1),
         lambda: K.encself_attention_i8qkv(q8_3h, b3h, 0.05, mask, None, ctx8, 30.0, BATCH, SEQ, h,
                                           d)),
    ]
    out = {}
    for name, nbytes, fn in cases:
        us = _queued_time_us(fn, reps)
        gbs = nbytes / (us * 1e-6) / 1e9
        out[name] = {"avg_us": us, "algorithmic_bytes": nbytes, "GB/s": gbs,
                     "frac_of_hbm_peak": gbs / HBM_PEAK_GBS}
    return out


_blocker = None


def _queued_time_us(fn, reps):
    """Average GPU time of ``fn``'s kernel over ``reps`` back-to-back launches.

    A host launch through ctypes costs more than these kernels run, so timing a plain loop
    measures the host.  A long matrix product is queued first; while it runs the host
    enqueues the start event, all the launches and the stop event, and the GPU then executes
    them back to back."""
    import torch
    global _blocker
    if _blocker is None:
        _blocker = torch.randn(8192, 8192, dtype=torch.float16, device="cuda:0")
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(4):
        torch.mm(_blocker, _blocker)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def gemm_microbench(reps=40):
    """The GEMM + fused dequant-bias-GELU-requant micro-benchmark: A 4096x1024 and W
    [4096, 1024] int8 uniform in [-127, 127], int32 output; the same product with the
    bias + GELU + requantisation in its epilogue (clips 4.0 / 0.08 / 6.0); the stand-alone
    int8 -> int8 bias-GELU kernel on the 4096x4096 output; and the 4096x4096 -> 1024 shape."""
    import torch
    from lightseq_amd import kernels as K
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(0)
    clip_in, clip_w, clip_out, clip_act = 4.0, 0.08, 6.0, 6.0
    out = {}
    for M, N, Kd in ((4096, 4096, 1024), (4096, 1024, 4096)):
        a = torch.randint(-127, 128, (M, Kd), dtype=torch.int8, device=dev, generator=g)
        w = torch.randint(-127, 128, (N, Kd), dtype=torch.int8, device=dev, generator=g)
        bias = (torch.randn(N, device=dev, generator=g) * 0.02).half()
        c32 = torch.zeros(M, N, dtype=torch.int32, device=dev)
        c8 = torch.zeros(M, N, dtype=torch.int8, device=dev)
        ops = 2.0 * M * N * Kd
        alpha = clip_in * clip_w / (clip_out * 127)
        lut = torch.zeros((N, 256), dtype=torch.int8, device=dev)
        K.build_act_lut(lut, bias, N, clip_out / 127, 127 / clip_act, clip_act, 0)
        cases = {
            "int32 out": lambda: K.gemm_i8_i32o(a, w, c32, M, N, Kd),
            "int8 out (requantising epilogue)": lambda: K.gemm_i8_i8o(a, w, c8, M, N, Kd, alpha),
            "int8 out, bias+GELU+requant fused": lambda: K.gemm_i8_bias_gelu_i8o(
                a, w, c8, bias, M, N, Kd, alpha, clip_out / 127, 127 / clip_act),
            "int8 out, bias+GELU+requant fused through the per-column table (what the models run; "
            "same bytes)": lambda: K.gemm_i8_lut_i8o(a, w, c8, lut, M, N, Kd, alpha),
        }
        res = {}
        for name, fn in cases.items():
            us = _queued_time_us(fn, reps)
            res[name] = {"avg_us": us, "TOP/s": ops / (us * 1e-6) / 1e12,
                         "frac_of_int8_mfma_peak": ops / (us * 1e-6) / 1e12 / INT8_MFMA_PEAK_TOPS}
        us = _queued_time_us(lambda: K.ker_bias_gelu_i8I_i8O_launcher(
            M, c8, c8, bias, N, clip_out / 127, 127 / clip_act), reps)
        nbytes = 2 * M * N
        res["stand-alone dequant-bias-GELU-requant i8->i8"] = {
            "avg_us": us, "algorithmic_bytes": nbytes, "GB/s": nbytes / (us * 1e-6) / 1e9,
            "frac_of_hbm_peak": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
        out["%dx%dx%d" % (M, N, Kd)] = res
    out["vendor_yardstick torch._int_mm (int32 out, same box; not used by the library)"] = _int_mm_yardstick(reps)
    out["large product 8192x8192x8192 (where launch, first-operand and write-back costs vanish)"] = \
        _large_product(max(reps // 4, 5))
    return out


def _large_product(reps):
    """The library's int8 GEMM and the vendor's on a product large enough that only the tile loop
    is timed: what the loop reaches on this box, and what the vendor's hand-tuned kernel does."""
    import torch
    from lightseq_amd import kernels as K
    dev = "cuda:0"
    M = N = Kd = 8192
    g = torch.Generator(device=dev).manual_seed(1)
    a = torch.randint(-127, 128, (M, Kd), dtype=torch.int8, device=dev, generator=g)
    w = torch.randint(-127, 128, (N, Kd), dtype=torch.int8, device=dev, generator=g)
    c8 = torch.zeros(M, N, dtype=torch.int8, device=dev)
    c32 = torch.zeros(M, N, dtype=torch.int32, device=dev)
    ops = 2.0 * M * N * Kd
    res = {}
    cases = {
        "int8 out (requantising epilogue)": lambda: K.gemm_i8_i8o(a, w, c8, M, N, Kd, 1e-4),
        "int32 out": lambda: K.gemm_i8_i32o(a, w, c32, M, N, Kd),
    }
    for name, fn in cases.items():
        us = _queued_time_us(fn, reps)
        res[name] = {"avg_us": us, "TOP/s": ops / (us * 1e-6) / 1e12,
                     "frac_of_int8_mfma_peak": ops / (us * 1e-6) / 1e12 / INT8_MFMA_PEAK_TOPS}
    try:
        wt = w.t()
        us = _queued_time_us(lambda: torch._int_mm(a, wt), reps)
        res["vendor torch._int_mm (int32 out)"] = {"avg_us": us, "TOP/s": ops / (us * 1e-6) / 1e12}
    except Exception as e:
        res["vendor torch._int_mm (int32 out)"] = {"error": repr(e)[:200]}
    return res


def _int_mm_yardstick(reps):
    """torch._int_mm (the vendor library's int8 GEMM as PyTorch-ROCm reaches it) on the layer's
    four products and the two micro-benchmark shapes, int32 output, timed like the rest."""
    import torch
    dev = "cuda:0"
    res = {}
    for M, N, Kd in ((4096, 2304, 768), (4096, 768, 768), (4096, 3072, 768), (4096, 768, 3072),
                     (4096, 4096, 1024), (4096, 1024, 4096)):
        key = "%dx%dx%d" % (M, N, Kd)
        try:
            a = torch.randint(-127, 128, (M, Kd), dtype=torch.int8, device=dev)
            b = torch.randint(-127, 128, (N, Kd), dtype=torch.int8, device=dev).t()
            us = _queued_time_us(lambda: torch._int_mm(a, b), reps)
            res[key] = {"avg_us": us, "TOP/s": 2.0 * M * N * Kd / (us * 1e-6) / 1e12}
        except Exception as e:  # record why the yardstick is missing
            res[key] = {"error": repr(e)[:200]}
    return res


TRAFFIC_SUMMARY = "bert_base_b32_s128_pmc_hbm_traffic.txt"


def _profiled_traffic(kernel, site):
    """HBM bytes per launch of ``kernel`` at GEMM site ``site`` from the committed
    rocprofv3 --pmc summary (FETCH_SIZE and WRITE_SIZE runs of this same command, scaled by
    a plain copy kernel); None when the summary holds no line for that kernel and site."""
    import re
    path = os.path.join(ROOT, "profiles", TRAFFIC_SUMMARY)
    if not os.path.exists(path):
        return None
    want = kernel.replace("EpiGeluI8", "EpiActI8<0>") + " @ " + site
    for line in open(path):
        m = re.match(r"traffic_bytes_per_launch\[(.+?)\] = (\d+)", line)
        if m and m.group(1).replace("lsh::", "") == want:
            return int(m.group(2))
    return None


def _per_step_event_times(model, steps):
    """Per-step GPU time between HIP events recorded on the model's own stream (a second pass
    over the same steps): median, 10th and 90th percentile, milliseconds."""
    import numpy as np
    import torch
    stream = torch.cuda.ExternalStream(model.get_stream())
    times = []
    for _ in range(steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        model.infer_device()
        e1.record(stream)
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    t = np.asarray(times)
    return {"median": float(np.median(t)), "p10": float(np.percentile(t, 10)),
            "p90": float(np.percentile(t, 90)), "steps": int(steps),
            "how": "HIP events on the model's stream around each Infer()"}


def _write_model(cfg):
    from lightseq_amd import synthetic
    tmp = tempfile.mkdtemp(prefix="ls_bench_")
    path = os.path.join(tmp, "quant_bert_base.pb")
    synthetic.write_quant_bert(path, cfg, seed=0)
    return path


def two_batches_in_flight(path_factory, steps):
    """Not the headline number: the same workload with two model instances (each with its own
    stream and buffers) driven by two host threads, so that two batches of 32 x 128 are in
    flight at once and the launch ramp and write-back of one instance's kernels overlap the
    other's compute.  Every step is still one Infer() over one batch."""
    import threading
    import torch
    from lightseq_amd import inference, synthetic
    cfg = synthetic.bert_config("bert_base")
    path = path_factory()
    ids, _ = synthetic.make_token_ids(cfg, BATCH, SEQ, seed=0, min_len=32)
    models = [inference.QuantBert(path, BATCH) for _ in range(2)]
    os.remove(path)
    for m in models:
        m._upload(ids)
        for _ in range(5):
            m.infer_device()
    torch.cuda.synchronize()

    def loop(m):
        for _ in range(steps):
            m.infer_device()
    threads = [threading.Thread(target=loop, args=(m,)) for m in models]
    t0 = time.perf_counter()
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for m in models:
        m.close()
    return {"value": 2 * BATCH * SEQ * steps / dt, "unit": "tokens/s", "instances": 2,
            "steps_per_instance": steps, "ms_per_step_per_instance": 1e3 * dt / steps,
            "what": "two QuantBert instances on two host threads, one Infer() per batch each"}


def bench_bert(args):
    import torch
    from lightseq_amd import inference, synthetic
    cfg = synthetic.bert_config("bert_base")
    tmp = tempfile.mkdtemp(prefix="ls_bench_")
    path = os.path.join(tmp, "quant_bert_base.pb")
    msg = synthetic.write_quant_bert(path, cfg, seed=0)
    ids, lens = synthetic.make_token_ids(cfg, BATCH, SEQ, seed=0, min_len=32)

    model = inference.QuantBert(path, BATCH)
    os.remove(path)
    model._upload(ids)  # token ids resident in HBM before the timed region

    for _ in range(args.warmup):
        model.infer_device()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        model.infer_device()  # synchronous: returns after the model's stream drained
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    tokens_per_s = BATCH * SEQ * args.steps / dt
    step_ms = _per_step_event_times(model, args.steps)

    # instrumented pass: HIP events around every int8 GEMM launch on the model's stream
    model.set_profiling(True)
    for _ in range(args.steps):
        model.infer_device()
    prof = model.get_profile()
    model.set_profiling(False)
    by_kernel = {}
    for site in prof:  # one entry per (instantiation, shape): a site has one shape
        k = by_kernel.setdefault((site["kernel"], site["site"]),
                                 {"ms": 0.0, "launches": 0, "ops": 0.0, "sites": []})
        k["ms"] += site["total_ms"]
        k["launches"] += site["launches"]
        ops = 2.0 * site["m"] * site["n"] * site["k"]
        if site["kernel"] == "ffn_segment_kernel":
            ops *= 2.0  # FFN1 and FFN2 in one launch: the same number of operations each
        if site["kernel"] == "qkv_attn_kernel":
            # the launch also holds the layer's attention: 4 B h S^2 d fp16 flops, counted
            # twice because the fp16 MFMA peak is half the int8 peak this is priced against
            # (the padded shape: the figure the fraction is quoted on; what the planned launch
            # executes after leaving out the blocks of padding is reported beside it)
            ops += 2.0 * 4.0 * BATCH * cfg["head_num"] * SEQ * SEQ * (cfg["hidden"] // cfg["head_num"])
        k["ops"] += ops * site["launches"]
        k["sites"].append(site["site"])
    (name, dom_site), dom = max(by_kernel.items(), key=lambda kv: kv[1]["ms"])
    avg_ms = dom["ms"] / dom["launches"]
    achieved = dom["ops"] / dom["launches"] / (avg_ms * 1e-3) / 1e12
    measured_peak = measured_mfma_peak()
    # what the fused QKV + attention launch executes with its plan: 32-token blocks that hold a token
    blocks = (lens + 31) // 32
    H_, h_ = cfg["hidden"], cfg["head_num"]
    executed_qkv = float((2.0 * 32 * blocks * 3 * H_ * H_).sum() +
                         2.0 * (4.0 * h_ * (32.0 * blocks) ** 2 * (H_ // h_)).sum())
    roofline = {"bound": "mfma", "achieved": achieved, "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOP/s",
                "frac": achieved / INT8_MFMA_PEAK_TOPS, "measured_peak": measured_peak,
                "frac_of_measured_peak": achieved / measured_peak,
                "measured_peak_how": "register-resident v_mfma_i32_32x32x32_i8 loop, 2 workgroups per "
                                     "compute unit (lsh_mfma_i8_peak_probe)",
                "ops_counted": ("2*M*N*K int8 operations of the product" +
                                (" + 2 x the 4*B*h*S^2*d fp16 flops of the attention in the same launch"
                                 if name == "qkv_attn_kernel" else "") +
                                (", FFN1 and FFN2 both (one launch; the layer norm in it adds none)"
                                 if name == "ffn_segment_kernel" else "")),
                "ops_executed": ({"per_launch": executed_qkv,
                                  "achieved": executed_qkv / (avg_ms * 1e-3) / 1e12,
                                  "what": "operations of the 32-token blocks that hold a token (valid "
                                          "lengths U[32,128]); `achieved` above counts the padded shape"}
                                 if name == "qkv_attn_kernel" else None),
                "traffic": _profiled_traffic(name, dom_site),
                "traffic_source": "profiles/" + TRAFFIC_SUMMARY, "kernel": name,
                "sites": dom["sites"], "avg_launch_us": avg_ms * 1e3,
                "gemm_sites": {s["site"]: {"kernel": s["kernel"], "mnk": [s["m"], s["n"], s["k"]],
                                           "avg_us": 1e3 * s["total_ms"] / max(1, s["launches"]),
                                           "tops": (2.0 if s["kernel"] == "ffn_segment_kernel" else 1.0)
                                           * 2.0 * s["m"] * s["n"] * s["k"] * s["launches"]
                                           / max(1e-12, s["total_ms"] * 1e-3) / 1e12}
                               for s in prof if s["launches"] > 0}}
    out = {
        "metric": "int8 tokens/sec BERT-base b32 s128; int8 GEMM % MFMA-i8 peak; fused GB/s",
        "value": tokens_per_s, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": 1e3 * dt / args.steps, "step_ms": step_ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "BERT-base-shaped int8 encoder stack: 12 layers, hidden 768, 12 heads, "
                               "FFN 3072 GELU, batch 32 x seq 128, valid lengths U[32,128] right-padded, "
                               "vocab 30522, random-init N(0,0.02) weights quantised per tensor",
                   "batch": BATCH, "seq_len": SEQ, "valid_tokens": int(lens.sum()),
                   "entry_point": "QuantBert / LSModel::Infer"},
        "roofline": roofline,
    }
    model.close()
    if not args.no_fused:
        out["two_batches_in_flight"] = two_batches_in_flight(path_factory=lambda: _write_model(cfg),
                                                             steps=args.steps)
        out["fused_kernels"] = fused_kernel_rates(cfg)
        out["fused_kernels_at_batch_512 (same kernels on 16 x the rows)"] = \
            fused_kernel_rates(cfg, reps=20, BATCH=512)
        out["gemm_microbench"] = gemm_microbench()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, msg, ids)
        out["cpu_baseline"]["torch_cpu"] = torch_cpu_baseline(cfg, ids)
    if not args.no_generation:
        # the two generation workloads, each a few whole Infer() calls (their own lines with
        # --workload): decode-step time against the HBM roofline, the oracle beside it
        out["generation"] = {w: bench_generation(w, steps=3, warmup=1, graphs=False,
                                                 with_cpu=not args.no_cpu_baseline)
                             for w in ("transformer_big", "gpt2_medium")}
    return out


def bench_ffn_segment(args):
    """A/B of the feed-forward half of a layer as one launch (rows dealt to the XCDs, XCD-local
    barriers; ``lsh_ffn_segment_i8_f16``) against its three launches, inside the BERT workload:
    step times of both routes, the event-timed launch, and the per-workgroup clock stamps at the
    kernel's phase boundaries."""
    import numpy as np
    import torch
    from lightseq_amd import inference, kernels as K, synthetic
    cfg = synthetic.bert_config("bert_base")
    path = _write_model(cfg)
    ids, _ = synthetic.make_token_ids(cfg, BATCH, SEQ, seed=0, min_len=32)
    model = inference.QuantBert(path, BATCH)
    os.remove(path)
    model._upload(ids)
    out = {"workload": "BERT-base b32 x s128, 12 layers", "ms_per_step": {}, "launch_us": {}}
    prev = K.ffn_segment_in_models(False)
    try:
        for rnd in range(3):
            for on in (True, False):
                K.ffn_segment_in_models(on)
                for _ in range(args.warmup):
                    model.infer_device()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    model.infer_device()
                torch.cuda.synchronize()
                out["ms_per_step"].setdefault("segment" if on else "three launches", []).append(
                    1e3 * (time.perf_counter() - t0) / args.steps)
        for on in (True, False):
            K.ffn_segment_in_models(on)
            model.set_profiling(True)
            for _ in range(args.steps):
                model.infer_device()
            prof = model.get_profile()
            model.set_profiling(False)
            out["launch_us"]["segment" if on else "three launches (the layer norm is not event-timed)"] = {
                p["site"]: {"kernel": p["kernel"], "avg_us": 1e3 * p["total_ms"] / p["launches"]}
                for p in prof if p["launches"] and p["site"] in ("ffn1", "ffn2")}
        K.ffn_segment_in_models(True)
        st = torch.zeros(256, 8, dtype=torch.int64, device="cuda:0")
        K.ffn_segment_stamps(st)
        runs = []
        for _ in range(20):
            model.infer_device()   # the stamps of the last layer's launch remain
            runs.append(st.cpu().numpy().copy())
        K.ffn_segment_stamps(None)
    finally:
        K.ffn_segment_in_models(prev)
    model.close()
    a = np.stack(runs).astype(np.float64) * 0.01  # 100 MHz clock -> microseconds
    names = ["start", "FFN1 done", "past barrier 1", "FFN2 done", "past barrier 2", "layer norm done"]
    d = np.diff(a, axis=2)
    out["phase_us (mean over the 256 workgroups; mean over launches of the slowest workgroup)"] = {
        "%s -> %s" % (names[i], names[i + 1]): [float(d[:, :, i].mean()), float(d[:, :, i].max(axis=1).mean())]
        for i in range(5)}
    out["first start -> last end, in-kernel, us"] = float((a[:, :, 5].max(axis=1) - a[:, :, 0].min(axis=1)).mean())
    return out


def _generation_setup(workload):
    """Model file, token ids and the shape figures of one generation workload."""
    import numpy as np
    from lightseq_amd import synthetic
    tmp = tempfile.mkdtemp(prefix="ls_bench_")
    if workload == "transformer_big":
        cfg = synthetic.transformer_config("transformer_big")
        src_len, steps_wanted, batch = 64, 64, 16
        # decoding runs min(max_step, src + extra) - 2 steps
        cfg.update(max_step=128, extra_decode_length=steps_wanted + 2 - src_len)
        path = os.path.join(tmp, "quant_transformer_big.pb")
        msg = synthetic.write_quant_transformer(path, cfg, seed=0)
        ids, _ = synthetic.make_token_ids(dict(vocab=cfg["src_vocab"], padding_id=0), batch, src_len,
                                          seed=0, min_len=src_len)
        desc = ("Transformer-big-shaped int8 encoder-decoder, beam search: hidden 1024, 16 heads, "
                "FFN 4096 ReLU, 6+6 layers, batch 16 x beam 4, source length 64, 64 decode steps, "
                "vocab 32000, random-init weights")
        return dict(cfg=cfg, msg=msg, path=path, ids=ids, batch=batch, src_len=src_len, desc=desc,
                    cls="QuantTransformer")
    cfg = synthetic.gpt_config("gpt2_medium")
    src_len, batch = 512, 16
    path = os.path.join(tmp, "quant_gpt2_medium.pb")
    msg = synthetic.write_quant_gpt(path, cfg, seed=0)
    ids = np.random.default_rng(0).integers(0, cfg["vocab"] - 1, size=(batch, src_len), dtype=np.int32)
    desc = ("GPT-2-medium-shaped int8 decoder-only generation: 24 layers, hidden 1024, 16 heads, "
            "FFN 4096 GELU, pre-LN, vocab 50257, batch 16, prompt 512, 128 generated tokens, "
            "greedy, random-init weights")
    return dict(cfg=cfg, msg=msg, path=path, ids=ids, batch=batch, src_len=src_len, desc=desc,
                cls="QuantGpt")


def _step_bytes(workload, cfg, batch, src_len, loop_steps):
    """Algorithmic HBM bytes of one decode step, averaged over the steps of the loop: every int8
    weight once, the cached keys and values the step's attention reads, the logits written and
    read once.  (The reference also copies the whole self-attention cache every step; no
    algorithm needs that and it is not counted.)"""
    H, I = cfg["hidden"], cfg["inner"]
    if workload == "transformer_big":
        L, V, rows = cfg["n_dec_layer"], cfg["trg_vocab"], batch * cfg["beam_size"]
        weights = L * (6 * H * H + 2 * H * I) + V * H
        avg_len = (loop_steps + 1) / 2.0                 # step t reads t + 1 cached positions
        cache = L * rows * 2 * H * avg_len               # int8 self-attention keys and values
        cross = L * batch * src_len * H * 2 * 2          # fp16 cross keys and values, once per sentence
    else:
        L, V, rows = cfg["n_layer"], cfg["vocab"], batch
        weights = L * 12 * H * H + V * H
        avg_len = src_len + 1 + (loop_steps + 1) / 2.0   # the first loop step reads prompt + 2 positions
        cache = L * rows * 2 * H * avg_len
        cross = 0
    logits = 2 * rows * V
    return {"weights": int(weights), "self_attention_cache": int(cache), "cross_attention_kv": int(cross),
            "logits": int(logits), "total": int(weights + cache + cross + logits)}


def _generation_cpu_baseline(workload, setup):
    """The C oracle on a bounded sample of the workload: the full width, depth and batch, a few
    decode steps.  Two runs that differ only in the number of steps; their difference prices a
    step without the encoder / prompt pass."""
    import numpy as np
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    cfg, msg, batch = setup["cfg"], setup["msg"], setup["batch"]
    few, more = 2, 6
    t_all = time.perf_counter()
    if workload == "transformer_big":
        from oracle import oracle
        from oracle.model_io import oracle_transformer_weights_from_message
        enc_w, dec_w = oracle_transformer_weights_from_message(msg, cfg, np.float16)
        ids = setup["ids"]
        enc_out, mask, _ = oracle.quant_bert_encoder(enc_w, ids)
        times, ran = [], []
        for n in (few, more):
            w = dict(dec_w, extra_decode_length=n + 2 - ids.shape[1])
            t0 = time.perf_counter()
            r = oracle.quant_decoder(w, enc_out, mask, is_benchmark=True)
            times.append(time.perf_counter() - t0)
            ran.append(r["steps_run"])
        what = "batch %d x beam %d, source %d" % (batch, cfg["beam_size"], ids.shape[1])
    else:
        from oracle import gpt
        w0 = gpt.gpt_weights_from_message(msg, cfg, np.float16)
        prompt = 32
        ids = setup["ids"][:, :prompt]
        times, ran = [], []
        for n in (few, more):
            w = dict(w0, extra_decode_length=n + 1)     # the prompt pass gives one token, the loop n
            t0 = time.perf_counter()
            r = gpt.quant_gpt_sample(w, ids, is_benchmark=True)
            times.append(time.perf_counter() - t0)
            ran.append(r["steps_run"])
        what = "batch %d, prompt cut to %d tokens (a step is priced by its weights)" % (batch, prompt)
    if ran[1] <= ran[0]:  # every sequence ended on its first token: nothing to price
        return {"value": None, "unit": "generated tokens/s (decode steps only)", "cores": cores,
                "kind": "port", "sample": "%s: the runs stopped after %s steps" % (what, ran)}
    per_step = (times[1] - times[0]) / (ran[1] - ran[0])
    return {"value": batch / per_step, "unit": "generated tokens/s (decode steps only)", "cores": cores,
            "kind": "port", "s_per_decode_step": per_step,
            "sample": "%s, full width and depth: runs of %d and %d decode steps, a step = their "
                      "difference / %d; %.1f s of CPU work" % (what, ran[0], ran[1], ran[1] - ran[0],
                                                               time.perf_counter() - t_all)}


def bench_generation(workload, steps, warmup, graphs=False, with_cpu=True):
    """Transformer-big beam search (batch 16 x beam 4, source 64, 64 steps) or
    GPT-2-medium greedy generation (batch 16, prompt 512, 128 new tokens): whole Infer() calls."""
    import numpy as np
    import torch
    from lightseq_amd import inference
    setup = _generation_setup(workload)
    cfg, batch, src_len, ids = setup["cfg"], setup["batch"], setup["src_len"], setup["ids"]
    model = getattr(inference, setup["cls"])(setup["path"], batch)
    os.remove(setup["path"])
    model.benchmark_mode(True)
    model._upload(ids)
    # launches of one step: the nodes of a captured step graph (two calls: keys seen, then captured)
    model.graph_mode(True)
    for _ in range(2):
        model.infer_device()
    launches = model.graph_nodes()
    model.graph_mode(bool(graphs))
    for _ in range(warmup):
        model.infer_device()
    torch.cuda.synchronize()
    prep, loop, nloop = [], [], 0
    t0 = time.perf_counter()
    for _ in range(steps):
        model.infer_device()
        a, b, nloop = model.phase_times()
        prep.append(a)
        loop.append(b)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    steps_run = model.steps_run()
    model.close()
    ms_step = float(np.mean(loop)) / max(1, nloop)
    nbytes = _step_bytes(workload, cfg, batch, src_len, nloop)
    gbs = nbytes["total"] / (ms_step * 1e-3) / 1e9
    out = {
        "metric": "generated tokens/sec (%s)" % workload,
        "value": batch * steps_run * steps / dt, "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": 1e3 * dt / steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": setup["desc"], "batch": batch, "source_len": src_len,
                   "generated_tokens_per_sequence": steps_run, "loop_steps": nloop,
                   "ms_before_the_step_loop": float(np.mean(prep)),
                   "ms_per_decode_step": ms_step, "launches_per_step": launches,
                   "us_per_launch": 1e3 * ms_step / max(1, launches),
                   "hip_graph_steps": bool(graphs),
                   "entry_point": setup["cls"] + " / LSModel::Infer",
                   "how": "wall clock around %d Infer() calls (value, ms_per_step); HIP events on the "
                          "model's stream around the step loop (ms_per_decode_step)" % steps},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "one decode step (%d dependent launches)" % launches,
                     "algorithmic_bytes_per_step": nbytes,
                     "launch_floor_frac": None},
    }
    if with_cpu:
        out["cpu_baseline"] = _generation_cpu_baseline(workload, setup)
    return out


def _leave():
    """Nothing may outlive the command: no helper thread or OpenMP team keeps the interpreter alive.  Under a
    profiler (rocprofv3 exports ROCP* variables) the process ends the ordinary way instead: the tool writes its
    files from exit handlers that os._exit would skip."""
    sys.stdout.flush()
    sys.stderr.flush()
    if any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ):
        return
    os._exit(0)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default="bert_base",
                    choices=["bert_base", "transformer_big", "gpt2_medium"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-fused", action="store_true",
                    help="skip the stand-alone timing of the fused kernels")
    ap.add_argument("--no-generation", action="store_true",
                    help="default workload: skip the two generation workloads of the `generation` block")
    ap.add_argument("--ffn-segment", action="store_true",
                    help="A/B and phase stamps of the one-launch feed-forward segment (not the headline line)")
    ap.add_argument("--graphs", action="store_true",
                    help="generation workloads: replay the steps as HIP graphs (ls_model_set_graph_mode)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 256 MiB device copies (dst = src + 1, one elementwise "
                         "kernel each), a kernel of known HBM traffic against which profiler byte "
                         "counters are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU only (every model object owns device 0 and "
                 "one stream, as in the reference); --gpus %d is not supported" % args.gpus)
    bert = args.workload == "bert_base"
    if args.steps is None:
        args.steps = 100 if bert else 3
    if args.warmup is None:
        args.warmup = 20 if bert else 1

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    if args.copy_calibration:
        # an elementwise kernel (not a copy engine): reads 256 MiB, writes 256 MiB
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
    if args.ffn_segment:
        print(json.dumps(bench_ffn_segment(args)))
        _leave()
        return
    out = bench_bert(args) if bert else bench_generation(args.workload, args.steps, args.warmup,
                                                         args.graphs, not args.no_cpu_baseline)
    print(json.dumps(out))
    _leave()


if __name__ == "__main__":
    main()
