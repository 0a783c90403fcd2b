#!/usr/bin/env python3
"""Benchmark of the fused LoRA SFT step on one MI355X.

A step is one sft_train_step (embedding gather, forward, cross-entropy, backward,
global-norm clip, AdamW) over one batch of synthetic tokens, with weights and
adapters resident in HBM.  Prints ONE JSON line: train tokens/s for the
Qwen3-4B-shaped LoRA r16 seq-64 F16 configuration, the weight-streaming GEMM's
achieved HBM bandwidth against the 8 TB/s peak (HIP events around every GEMM
launch on the library's stream), and the CPU oracle timed on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from llm_metal_amd.configs import CONFIGS  # noqa: E402
from llm_metal_amd.synth import make_batch, make_model  # noqa: E402

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFS = 2500.0          # dense fp16 MFMA


TRAFFIC_SUMMARIES = {"c3_qwen3_4b_f16": ("c3_gemm_hbm_traffic_pmc.txt", "c3"),
                     "c3_qwen3_4b_q8_seq64": ("c3_q8_step_trace_and_hbm_traffic.txt", "c3q"),
                     "c2_gemma3_1b": ("c2_gemm_hbm_traffic_pmc.txt", "c2"),
                     "c4_qwen3_4b_q8": ("c4_gemm_hbm_traffic_pmc.txt", "c4"),
                     "c5_gemma3_1b_grpo": ("c5_step_hbm_traffic_pmc.txt", "c5")}


def measured_traffic(cfg_name, kernels):
    """HBM bytes per timed launch from the committed hardware-counter summary of this workload (two rocprofv3
    --pmc runs, FETCH_SIZE and WRITE_SIZE, scaled by a copy kernel of known size), or None when there is none, or when
    the summary was made for another kernel than the one that runs now (its `traffic_kernel_*` line)."""
    if cfg_name not in TRAFFIC_SUMMARIES:
        return None
    name, tag = TRAFFIC_SUMMARIES[cfg_name]
    path = os.path.join(ROOT, "profiles", name)
    if not os.path.exists(path):
        return None
    value, kernel = None, None
    for line in open(path):
        if line.startswith(f"traffic_bytes_per_gemm_launch_{tag}"):
            value = float(line.split("=")[1])
        if line.startswith(f"traffic_kernel_{tag}"):
            kernel = line.split("=")[1].strip()
    if kernel is not None and kernel not in kernels:
        return None
    return value


def gemm_shapes(cfg, L):
    """One line per product shape of a LoRA step at cfg.BN rows (F16 weights): microseconds per launch, launched back to
    back on the library's stream with the weights rotated through more than 1 GB (nothing is found in a cache), for
    (a) the weight loads of gemm_ring alone on its grid, (b) gemm_ring or, where the planner takes it, gemm_ring_wide (named in
    `ring_kernel`), (c) gemm_tiled; and a fit  t = t0 + bytes / rate
    over the layer shapes.  An empty kernel launched the same way takes about 3 us, which every figure includes."""
    import ctypes as C
    D, qd, kd, IS, V, R = cfg.D, cfg.Hq * cfg.hd, cfg.Hkv * cfg.hd, cfg.IS, cfg.V, cfg.R
    nq = qd + 2 * kd + 2 * R
    shapes = [("qkv forward", nq, D), ("o forward", D, qd), ("gate|up forward", 2 * IS, D), ("down forward", D, IS),
              ("down backward", IS, D), ("gate|up backward", D, 2 * IS), ("o backward", qd, D), ("qkv backward", D, nq),
              ("lm_head forward", V, D), ("lm_head backward", D, V)]
    rows = []
    for name, N, K in shapes:
        nb, S = C.c_int(0), C.c_int(0)
        it = 20 if N * K > 2e8 else 100
        L.hip_gemm_ring(1)
        t_read = L.hip_gemm_time_shape(cfg.BN, N, K, -1, 0, 0, it, C.byref(nb), C.byref(S)) * 1e3
        t_ring = L.hip_gemm_time_shape(cfg.BN, N, K, 0, 0, 0, it, C.byref(nb), C.byref(S)) * 1e3
        s_ring, wide = S.value, nb.value == 4
        L.hip_gemm_ring(0)
        t_tiled = L.hip_gemm_time_shape(cfg.BN, N, K, 0, 0, 0, it, C.byref(nb), C.byref(S)) * 1e3
        s_tiled = S.value
        L.hip_gemm_ring(1)
        mb = 2.0 * N * K / 1e6
        rows.append({"product": name, "N": N, "K": K, "MB": round(mb, 1), "weights_only_us": round(t_read, 2), "gemm_ring_us": round(t_ring, 2),
                     "ring_chunks": s_ring, "ring_kernel": "gemm_ring_wide" if wide else "gemm_ring", "gemm_tiled_us": round(t_tiled, 2), "tiled_chunks": s_tiled,
                     "weights_only_GBs": round(mb / t_read * 1e3), "gemm_ring_GBs": round(mb / t_ring * 1e3), "gemm_tiled_GBs": round(mb / t_tiled * 1e3)})
    layer = rows[:8]
    x = np.array([r["MB"] for r in layer]); fits = {}
    for key in ("weights_only_us", "gemm_ring_us", "gemm_tiled_us"):
        y = np.array([r[key] for r in layer])
        slope, t0 = np.polyfit(x, y, 1)
        fits[key] = {"t0_us": round(float(t0), 2), "rate_GBs": round(1e3 / float(slope))}
    emit({"workload": cfg.name, "rows": cfg.BN, "shapes": rows, "fit_over_layer_shapes": fits})


def cpu_baseline(cfg, budget_s=20.0):
    """Times the CPU oracle (scalar port of the reference's arithmetic, 1 thread) on a bounded
    sample of the same workload: the full step on a model with fewer layers and a truncated
    vocabulary, scaled to the full configuration by the GEMM flop ratio."""
    from oracle import oracle
    nl = min(cfg.NL, 3)
    v = min(cfg.V, 16384)
    small = cfg.with_(name=cfg.name + "_sample", NL=nl, V=v, tied=False)
    model = make_model(small, seed=0)
    used = oracle.weights_as_used(model)
    tok, tgt = make_batch(small, seed=1)
    lora = model["lora"].copy()
    m, vv = np.zeros_like(lora), np.zeros_like(lora)
    t0 = time.perf_counter()
    if cfg.R:
        oracle.sft_train_step(small, used, lora, m, vv, 0, tok, tgt, 1e-4)
    else:                                                  # full-parameter: forward + backward with F16 gradient accumulation
        oracle.full_param_pass(small, used, oracle.new_grad_accum(used), tok=tok, tgt=tgt)
    dt = time.perf_counter() - t0
    scale = cfg.frozen_params / small.frozen_params
    est = dt * scale
    return {"value": cfg.BN / est, "unit": "tokens/s", "cores": 1, "host_cores_total": os.cpu_count(), "kind": "port",
            "sample": f"oracle full step on {nl} of {cfg.NL} layers + {v} of {cfg.V} vocab rows "
                      f"({dt:.1f} s measured), scaled by the frozen-parameter ratio {scale:.1f}; one thread "
                      f"(the reference's CPU path has no threading) of the box's {os.cpu_count()} logical cores"}


def decode_cpu_baseline(cfg):
    """The CPU oracle's decode chain (scalar, 1 thread) for one token at position 16 on a model with fewer layers
    and a truncated vocabulary, scaled to the full configuration by the frozen-parameter ratio."""
    from oracle import oracle
    from oracle.oracle import op
    nl, v = min(cfg.NL, 8), min(cfg.V, 32768)
    small = cfg.with_(name=cfg.name + "_sample", NL=nl, V=v, tied=False)
    model = make_model(small, seed=0)
    from llm_metal_amd.synth import MATS
    mats = [model[k][L] for L in range(nl) for k in MATS] + [model["lm_head"]]
    W = [np.ascontiguousarray(m.astype(np.float16)).view(np.uint16) for m in mats]
    x = np.ones(max(small.D, small.IS, small.Hq * small.hd), np.float32)
    y = np.zeros(max(small.V, small.IS), np.float32)
    t0 = time.perf_counter()
    for w in W:                                            # the products are all but a per-mille of a decode step's work
        op("f32", "or_f16_batch_matvec", w, x, y, w.shape[0], w.shape[1], 1)
    dt = time.perf_counter() - t0
    scale = cfg.frozen_params / small.frozen_params
    return {"value": 1.0 / (dt * scale), "unit": "tokens/s", "cores": 1, "host_cores_total": os.cpu_count(), "kind": "port",
            "sample": f"oracle matrix-vector products of one token on {nl} of {cfg.NL} layers + {v} of {cfg.V} vocab rows "
                      f"({dt:.2f} s measured), scaled by the frozen-parameter ratio {scale:.1f}"}


def decode_bench(args, cfg, L):
    """Greedy generation, one token per step; the matrix-vector kernel is the dominant kernel and every one of its
    launches is timed with HIP events on the library's stream in a second pass."""
    import ctypes as C
    from llm_metal_amd.sft import InferenceState, SFTState
    f16 = cfg.weight_format == "f16"
    t0 = time.perf_counter()
    model = make_model(cfg, seed=0)
    t_gen = time.perf_counter() - t0
    max_seq = args.prompt_len + args.warmup + 2 * args.steps + 8
    sft = None
    if args.decode_from_sft:                               # the generation state reads the training state's tiles in place
        sft = SFTState(cfg, model)
        inf = InferenceState(sft=sft, max_seq=max_seq)
    else:
        inf = InferenceState(cfg, model, max_seq=max_seq, use_fp16=f16)
    t_init = time.perf_counter() - t0 - t_gen
    del model
    rng = np.random.default_rng(3)
    tok = 1
    for t in rng.integers(0, cfg.V, args.prompt_len):
        tok = inf.forward_token_argmax(int(t))
    for _ in range(args.warmup):
        tok = inf.forward_token_argmax(tok)
    L.metal_flush()
    t1 = time.perf_counter()
    for _ in range(args.steps):
        tok = inf.forward_token_argmax(tok)
    L.metal_flush()
    dt = time.perf_counter() - t1
    prof_steps = max(1, min(5, args.steps))
    L.hip_gemm_profile_enable(1)
    for _ in range(prof_steps):
        tok = inf.forward_token_argmax(tok)
    tms, wb, fl = C.c_double(0), C.c_double(0), C.c_double(0)
    n = L.hip_gemm_profile_read2(C.byref(tms), C.byref(wb), C.byref(fl))
    L.hip_gemm_profile_enable(0)
    batch = None
    if args.decode_batch > 1 and (f16 or sft is not None):
        # the same prompt decoded in lock step by `decode_batch` copies (qwen3_generate_fast_batch); a never-emitted EOS id
        # keeps every copy going; the timed call includes the prefill of its prompt
        inf.set_eos([cfg.V + 1])
        prompt = rng.integers(1, cfg.V, args.prompt_len).astype(np.uint32)
        inf.generate_batch(prompt, 2, args.decode_batch)               # builds the tiled weight images and the caches once
        tb = time.perf_counter()
        got = inf.generate_batch(prompt, args.steps, args.decode_batch)
        dtb = time.perf_counter() - tb
        steps_b = args.prompt_len + got.shape[1] - 1
        batch = {"batch": args.decode_batch, "ms_per_step": round(dtb / steps_b * 1e3, 3),
                 "tokens_per_s": round(args.decode_batch * steps_b / dtb, 1), "steps": steps_b}
    inf.free()
    if sft is not None:
        sft.free()
    gbs = wb.value / (tms.value * 1e-3) / 1e9 if tms.value > 0 else 0.0
    out = {"metric": "greedy decode tokens/s, batch 1", "value": round(args.steps / dt, 1), "unit": "tokens/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(dt / args.steps * 1e3, 3), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "f16 weights x f32 activations, f32 accumulate" if f16 else
           "q8_0 weights x f32 activations, f32 accumulate", "data": "synthetic",
           "config": {"workload": cfg.name + "_decode", "layers": cfg.NL, "frozen_params": cfg.frozen_params,
                      "weight_format": cfg.weight_format, "prompt_len": args.prompt_len,
                      "weights": "own row-major matrices" if sft is None else "the training state's tiles, read in place"},
           "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                        "kernel": "k_matvec" if sft is None else "gemm_ring",
                        "launches_per_step": n // prof_steps, "avg_launch_us": round(tms.value * 1e3 / max(n, 1), 2),
                        "weight_bytes_per_step": wb.value / prof_steps, "matvec_ms_per_step": round(tms.value / prof_steps, 3)},
           "setup_s": {"generate_weights": round(t_gen, 1), "upload_convert": round(t_init, 1)}}
    if batch:
        out["batched"] = batch
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = decode_cpu_baseline(cfg)
    emit(out)


class _LibraryStdoutToStderr:
    """The library reports like the reference does, with printf on stdout ("[FastSFT] Grad accum buffers allocated ...").
    While this is active, file descriptor 1 is stderr, so that the one JSON line is all this program writes to stdout."""

    def __enter__(self):
        import ctypes
        self.libc = ctypes.CDLL(None)
        sys.stdout.flush()
        self.saved = os.dup(1)
        os.dup2(2, 1)
        return self

    def __exit__(self, *exc):
        self.libc.fflush(None)
        sys.stdout.flush()
        os.dup2(self.saved, 1)
        os.close(self.saved)


def emit(obj):
    """The result line, on the real stdout."""
    line = json.dumps(obj)
    if _REAL_STDOUT is not None:
        os.write(_REAL_STDOUT, (line + "\n").encode())
    else:
        print(line)


_REAL_STDOUT = None


def main():
    global _REAL_STDOUT
    with _LibraryStdoutToStderr() as redirect:
        _REAL_STDOUT = redirect.saved
        try:
            return _main()
        finally:
            _REAL_STDOUT = None


def _main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default: 200 training steps, or 20 decoded tokens with --decode)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default: 20, or 3 with --decode)")
    ap.add_argument("--config", default="c3_qwen3_4b_f16")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--seq", type=int, default=0, help="override the configuration's sequence length (experiments only)")
    ap.add_argument("--batch", type=int, default=0, help="override the configuration's batch (experiments only)")
    ap.add_argument("--q8-large-m", choices=("kept-image", "image-per-product", "unpack-in-lds"), default="kept-image",
                    help="how products with >= 1024 rows read Q8_0 weights: the F16 image a state keeps once made (default), "
                         "an F16 image made for every product, or Q8_0 tiles unpacked into LDS by the GEMM itself")
    ap.add_argument("--attn-bwd-one-launch", type=int, choices=(0, 1), default=1,
                    help="0: up to 64 positions too, the attention backward is two launches (dQ, then dK / dV) (comparisons only)")
    ap.add_argument("--half-planes", type=int, choices=(0, 1), default=1,
                    help="0: fp32 K-split planes for every product (comparisons only)")
    ap.add_argument("--gemm-ring-wide", type=int, choices=(0, 1), default=1,
                    help="1: gemm_ring_wide (four weight row blocks per workgroup) where the product has the row tiles for it")
    ap.add_argument("--gemm-ring", type=int, choices=(0, 1), default=1,
                    help="0: the products of up to 64 rows take the register-staged streaming kernel (gemm_tiled) instead of gemm_ring (comparisons only)")
    ap.add_argument("--attention", choices=("auto", "flash", "saved-probs"), default="auto",
                    help="training attention kernels: by the measured rule (default), without / with saved probabilities")
    ap.add_argument("--decode", action="store_true",
                    help="time greedy token-by-token generation (include/inference_hip.h) on the configuration's model "
                         "instead of the training step: a step is one token")
    ap.add_argument("--prompt-len", type=int, default=16)
    ap.add_argument("--decode-from-sft", action="store_true",
                    help="with --decode: a generation state made from a training state (inference_state_create_from_sft)")
    ap.add_argument("--decode-batch", type=int, default=0,
                    help="with --decode: also time this many copies of one prompt decoded in lock step")
    ap.add_argument("--gemm-shapes", action="store_true",
                    help="time every product shape of the configuration alone, with cold weights: the weight loads only, gemm_ring, gemm_tiled")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run the library's plain copy kernel (1 GiB in, 1 GiB out, 5 launches): "
                         "the known-size reference for scaling FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.steps is None:
        args.steps = 20 if args.decode else 200
    if args.warmup is None:
        args.warmup = 3 if args.decode else 20
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the step has no multi-GPU path); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    cfg = CONFIGS[args.config]
    if args.seq or args.batch:
        cfg = cfg.with_(seq=args.seq or cfg.seq, batch=args.batch or cfg.batch)

    from llm_metal_amd import lib
    from llm_metal_amd.sft import SFTState
    L = lib.load()

    if args.copy_calibration:
        if L.fast_metal_init() != 0:
            sys.exit("no gfx950 device")
        n = 1 << 28                                        # floats: 1 GiB read + 1 GiB written per launch
        src, dst = L.metal_buf_create(4 * n), L.metal_buf_create(4 * n)
        L.metal_enqueue_scale(src, 0.0, n)                 # touch the source once
        for _ in range(5):
            L.metal_enqueue_copy(src, dst, n)
        L.metal_flush()
        L.metal_buf_free(src), L.metal_buf_free(dst)
        L.fast_metal_shutdown()
        emit({"copy_calibration": {"kernel": "k_copy", "bytes_read_per_launch": 4 * n,
                                   "bytes_written_per_launch": 4 * n, "launches": 5}})
        return

    if args.decode:
        return decode_bench(args, cfg, L)
    if args.gemm_shapes:
        return gemm_shapes(cfg, L)

    t0 = time.perf_counter()
    model = make_model(cfg, seed=0, lora_b_std=0.0)          # timing runs: B = 0 as the reference initialises it
    t_gen = time.perf_counter() - t0
    L.hip_attention_flash({"auto": -1, "flash": 1, "saved-probs": 0}[args.attention])
    L.hip_gemm_ring(args.gemm_ring)
    L.hip_gemm_ring_wide(args.gemm_ring_wide)
    L.hip_gemm_half_planes(args.half_planes)
    L.hip_attention_backward_one_launch(args.attn_bwd_one_launch)
    if args.q8_large_m == "image-per-product":
        L.hip_gemm_image_budget_mb(0)
    elif args.q8_large_m == "unpack-in-lds" and cfg.weight_format != "f16" and cfg.BN >= 1024:
        L.hip_gemm_force_large_m(2)
    st = SFTState(cfg, model)
    t_init = time.perf_counter() - t0 - t_gen
    del model
    batches = [make_batch(cfg, seed=100 + i) for i in range(4)]
    lr = 1e-4

    grpo = cfg.R == 0
    if grpo:
        # GRPO phases 3-4 (src/nn/fast_grpo.c:376-495): 4 completions of 128 tokens after a 32-token prompt,
        # group-normalised N(0,1) advantages, old log-probabilities = the policy's own (ratio 1, clip inactive)
        rng = np.random.default_rng(7)
        G, p_len = 4, 32
        prompt = rng.integers(0, cfg.V, p_len).astype(np.uint32)
        comps = [rng.integers(0, cfg.V, cfg.seq - p_len).astype(np.uint32) for _ in range(G)]
        r = rng.standard_normal(G).astype(np.float32)
        adv = (r - r.mean()) / (r.std() + 1e-8)
        zeros = [np.zeros(cfg.seq - p_len, dtype=np.float32) for _ in range(G)]
        new_lp = st.grpo_apply_completions(prompt, comps, zeros, np.zeros(G, dtype=np.float32), 0.2, 0.0)
        old = [new_lp[i, p_len:].copy() for i in range(G)]
        lr = 1e-5
        step = lambda i: st.grpo_apply_completions(prompt, comps, old, adv, 0.2, lr)
        rows_per_step = G * cfg.seq
    else:
        step = lambda i: st.train_step(*batches[i % 4], lr)
        rows_per_step = cfg.BN
    for i in range(args.warmup):
        step(i)
    L.metal_flush()
    t1 = time.perf_counter()
    loss = 0.0
    for i in range(args.steps):
        loss = step(i)
    L.metal_flush()
    dt = time.perf_counter() - t1
    ms = dt / args.steps * 1e3
    toks = rows_per_step * args.steps / dt
    if grpo:
        loss = float(np.mean(loss[:, 32:]))                # mean log-probability of the sampled tokens

    # dominant kernel: the weight-streaming GEMM, timed launch by launch with HIP events on the library's stream
    prof_steps = max(1, min(20, args.steps))
    L.hip_gemm_profile_enable(1)
    for i in range(prof_steps):
        step(i)
    import ctypes as C
    tms, wb, fl = C.c_double(0), C.c_double(0), C.c_double(0)
    n = L.hip_gemm_profile_read2(C.byref(tms), C.byref(wb), C.byref(fl))
    L.hip_gemm_profile_enable(0)
    gbs = wb.value / (tms.value * 1e-3) / 1e9 if tms.value > 0 else 0.0
    tfs = fl.value / (tms.value * 1e-3) / 1e12 if tms.value > 0 else 0.0
    # the GEMMs stream every weight once per pass; from a few hundred rows on their flops, not the bytes, bound them
    # (ridge of the MI355X: 2.5 PFLOP/s / 8 TB/s = 312 flop per byte = 156 rows of F16 weights, 83 rows of Q8_0)
    compute_bound = fl.value / max(wb.value, 1.0) > MFMA_PEAK_TFS * 1e12 / (HBM_PEAK_GBS * 1e9)
    roofline = {"bound": "mfma" if compute_bound else "hbm",
                "achieved": round(tfs if compute_bound else gbs, 1),
                "peak": MFMA_PEAK_TFS if compute_bound else HBM_PEAK_GBS,
                "unit": "TFLOP/s" if compute_bound else "GB/s",
                "frac": round(tfs / MFMA_PEAK_TFS if compute_bound else gbs / HBM_PEAK_GBS, 4), "traffic": None,
                "kernel": ("gemm_big_q8<1>, gemm_big_q8<2>" if cfg.BN >= 1024 and cfg.weight_format != "f16" and args.q8_large_m == "unpack-in-lds" else
                           "gemm_big_f16_256, gemm_big_f16" if cfg.BN >= 1024 else
                           # full-parameter pass: the products, the weight gradients (F16 read-modify-write of the accumulators), the
                           # apply (W, G and the transposed image) and the operand transposes (time only) are timed together
                           "gemm_tiled, gemm_big_f16*, k_wgrad, k_apply_retile, k_transpose_scaled_jobs" if cfg.R == 0 else
                           "gemm_ring, gemm_ring_wide" if 32 < cfg.BN <= 64 and args.gemm_ring and args.gemm_ring_wide else
                           "gemm_ring" if cfg.BN <= 64 and args.gemm_ring else "gemm_tiled"),
                "launches_per_step": n // prof_steps,
                "avg_launch_us": round(tms.value * 1e3 / max(n, 1), 2),
                "weight_bytes_per_step": wb.value / prof_steps, "flop_per_step": fl.value / prof_steps,
                "gemm_ms_per_step": round(tms.value / prof_steps, 3)}
    roofline["traffic"] = measured_traffic(cfg.name, roofline["kernel"])
    roofline["traffic_source"] = (f"profiles/{TRAFFIC_SUMMARIES.get(cfg.name, ('',))[0]}: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, "
                                  "scaled by the same counters on a copy kernel of known size; not re-measured in this run"
                                  if roofline["traffic"] is not None else "no hardware-counter summary of the kernel that runs now is committed for this workload")
    st.free()

    metric = ("SFT train tokens/s, Qwen3-4B LoRA r16 seq64; % of HBM-BW / MFMA peak" if cfg.name == "c3_qwen3_4b_f16" else
              "GRPO train tokens/s, full-parameter F16 accumulate + apply" if grpo else "SFT train tokens/s")
    out = {"metric": metric,
           "value": round(toks, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(ms, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": ("q8_0 weights unpacked to f16 in LDS x f16 activations, f32 accumulate"
                     if cfg.weight_format != "f16" and cfg.BN >= 1024 and args.q8_large_m == "unpack-in-lds" else
                     "q8_0 weights as f16 images x f16 activations, f32 accumulate" if cfg.weight_format != "f16" and cfg.BN >= 1024 else
                     "q8_0 weights unpacked to f16 in LDS x f16 activations, f32 accumulate (the K-chunk sums of five products per layer leave as f16)"
                     if cfg.weight_format != "f16" and cfg.BN <= 64 and args.gemm_ring and args.half_planes and cfg.R > 0 else
                     "q8_0 weights unpacked to f16 in LDS x f16 activations, f32 accumulate" if cfg.weight_format != "f16" and cfg.BN <= 64 and args.gemm_ring else
                     "q8_0 weights unpacked to f16 in registers x f16 activations, f32 accumulate" if cfg.weight_format != "f16" else
                     "f16 weights x f16 activations, f32 accumulate (the K-chunk sums of five products per layer leave as f16)"
                     if cfg.R > 0 and cfg.BN <= 64 and args.half_planes and args.gemm_ring else
                     "f16 weights x f16 activations, f32 accumulate"), "data": "synthetic",
           "config": {"workload": cfg.name, "rows_per_step": rows_per_step, "layers": cfg.NL, "lora_rank": cfg.R,
                      "frozen_params": cfg.frozen_params, "weight_format": cfg.weight_format,
                      **({"q8_large_m": args.q8_large_m} if cfg.weight_format != "f16" and cfg.BN >= 1024 else {})},
           "roofline": roofline, "final_loss": round(float(loss), 5),
           "setup_s": {"generate_weights": round(t_gen, 1), "upload_convert": round(t_init, 1)}}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg)
    emit(out)


if __name__ == "__main__":
    main()
