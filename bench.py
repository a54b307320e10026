#!/usr/bin/env python3
"""Benchmark of the int8 transformer-layer forward path on one MI355X.

Workload: the BERT-base-shaped int8 encoder stack --
12 layers, hidden 768, 12 heads, FFN 3072 GELU, batch 32 x max seq 128, per-sequence
valid lengths uniform in [32, 128] with right padding, token ids uniform over a
30522 vocabulary, random-init weights ~N(0, 0.02) quantised per tensor -- run
through the drop-in entry point ``QuantBert(path, max_batch)`` / ``LSModel::Infer``.
A step is one ``Infer()`` over one batch whose token ids are already resident in
HBM.  ``value`` = batch * seq_len * steps / wall time of the timed steps (padded
tokens counted, as the reference's b32 x s128 figures do).

The JSON line also carries
  roofline      the dominant kernel (by total time) among the int8 GEMM
                instantiations, timed with HIP events on the model's stream during a
                second, instrumented pass over the same steps: achieved = 2*M*N*K per
                launch / mean launch time, against the 5.0 POP/s dense int8 MFMA peak;
  cpu_baseline  the CPU oracle (a C port of the reference's algorithm, OpenMP) timed
                on this host on a bounded sample of the same workload.
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

BATCH, SEQ = 32, 128


def cpu_baseline(cfg, msg, ids, layers=12):
    """Oracle timed on the host: `layers` encoder layers of the real width at the full
    b32 x s128 batch, scaled to the 12-layer stack."""
    import numpy as np
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
            "sample": "one step: %d of %d encoder layers at batch %d x seq %d, %.1f s of CPU work%s"
                      % (layers, cfg["n_layer"], ids.shape[0], ids.shape[1], dt,
                         "" if layers == cfg["n_layer"] else ", scaled to the full stack")}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU only (every model object owns device 0 and "
                 "one stream, as in the reference); --gpus %d is not supported" % args.gpus)

    import torch
    from lightseq_amd import inference, synthetic

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
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

    # instrumented pass: HIP events around every int8 GEMM launch on the model's stream
    model.set_profiling(True)
    for _ in range(args.steps):
        model.infer_device()
    prof = model.get_profile()
    model.set_profiling(False)
    by_kernel = {}
    for site in prof:
        k = by_kernel.setdefault(site["kernel"], {"ms": 0.0, "launches": 0, "ops": 0.0, "sites": []})
        k["ms"] += site["total_ms"]
        k["launches"] += site["launches"]
        k["ops"] += 2.0 * site["m"] * site["n"] * site["k"] * site["launches"]
        k["sites"].append(site["site"])
    name, dom = max(by_kernel.items(), key=lambda kv: kv[1]["ms"])
    avg_ms = dom["ms"] / dom["launches"]
    achieved = dom["ops"] / dom["launches"] / (avg_ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "achieved": achieved, "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOP/s",
                "frac": achieved / INT8_MFMA_PEAK_TOPS, "traffic": None, "kernel": name,
                "sites": dom["sites"], "avg_launch_us": avg_ms * 1e3,
                "gemm_sites": {s["site"]: {"kernel": s["kernel"], "mnk": [s["m"], s["n"], s["k"]],
                                           "avg_us": 1e3 * s["total_ms"] / max(1, s["launches"]),
                                           "tops": 2.0 * s["m"] * s["n"] * s["k"] * s["launches"]
                                           / max(1e-12, s["total_ms"] * 1e-3) / 1e12}
                               for s in prof}}

    out = {
        "metric": "int8 tokens/sec BERT-base b32 s128; int8 GEMM % MFMA-i8 peak; fused GB/s",
        "value": tokens_per_s, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": 1e3 * dt / args.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "BERT-base-shaped int8 encoder stack: 12 layers, hidden 768, 12 heads, "
                               "FFN 3072 GELU, batch 32 x seq 128, valid lengths U[32,128] right-padded, "
                               "vocab 30522, random-init N(0,0.02) weights quantised per tensor",
                   "batch": BATCH, "seq_len": SEQ, "valid_tokens": int(lens.sum()),
                   "entry_point": "QuantBert / LSModel::Infer"},
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, msg, ids)
    model.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
