#!/usr/bin/env python3
"""Decode throughput of the HIP PTIR backend on one MI355X.

Workload (BASELINE.json configs[3], batch 1): Ministral-3B-shaped decoder, bf16 weights and matmul
operands with an f32 residual stream and f32 logits (`--residual bf16`: every tensor bf16),
random-init N(0, 0.02) weights from a seed, prompt of 1024 random token ids, greedy decode with a
fixed-capacity KV cache.  One "step" = one decode token: upload of the per-step scalars, one
`run_program` over the whole model, on-device argmax and the 8-byte token readback -- the
reference's decode-steady protocol (crates/gpt-rs-cli/src/main.rs:976-1051).

Prints ONE JSON line; `value` = tokens/s with all weights and the KV cache resident in HBM.
`roofline` covers the dominant kernel, the persistent decode chain (one launch per step: every
linear layer and the decode attention): the step's algorithmic bytes (every weight element once,
the valid KV rows once, activations and logits once) over the HIP-event time of those launches on
the backend's stream.  `prefill` prices the 1024-token prefill against the bf16 MFMA peak, `gpt2_f32`
is the other half of the metric (GPT-2 small f32: whole generate calls of 64 tokens, and steady
decode against the HBM roofline).  `cpu_baseline` (and `gpt2_f32.cpu_baseline`) time the reference C
backend's own kernels (oracle/_ref, built from the reference checkout) on the host, before the GPU
is touched: one core, the reference's own setting, and one process per core.
"""
from __future__ import annotations

import argparse
import ctypes
import hashlib
import json
import os
import struct
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBPS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
# HBM bytes moved by one chain_kernel launch of the default workload (26 layers, prompt 1024, cache length ~1040), from
# rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a copy kernel of known size (commands and raw figures: `profile`).  The
# figure belongs to ONE version of the kernel: `source_sha256` is the hash of gpt.rs_amd/csrc/kernels_chain.hip it was
# measured on, and `roofline.traffic` is null whenever the file in the tree hashes differently.
CHAIN_TRAFFIC = {"bytes": 7.0149e9 + 0.0273e9, "w8_bytes": 3.5937e9 + 0.0274e9,
                 "source_sha256": "ed3ebc9b622d507ae693373ec872176c091fc4e53d7ff9f3f93152d1901b2a42",
                 "profile": "profiles/chain_kernel_ministral3b_bf16_b1_decode.md"}


def chain_traffic_bytes(key: str = "bytes"):
    try:
        with open(os.path.join(ROOT, "gpt.rs_amd", "csrc", "kernels_chain.hip"), "rb") as f:
            return CHAIN_TRAFFIC[key] if hashlib.sha256(f.read()).hexdigest() == CHAIN_TRAFFIC["source_sha256"] else None
    except OSError:
        return None


def algorithmic_bytes_per_step(cfg, dtype_bytes: int, cache_len: int, quant: str = "none", f32_stream: bool = False) -> int:
    """Minimum HBM traffic of one decode token: every weight once, the valid KV once, the new KV
    row and the logits written once.  Quantised linear weights count their codes (1 or 1/2 byte per
    element) plus their scales (one per column, or one per column and 128 rows).  f32_stream: norm
    gains and logits are f32."""
    a = cfg.attention_config()
    mats = cfg.num_layers * [(cfg.embed_dim, a.total_projection_dim), (a.query_projection_dim, cfg.embed_dim),
                             (cfg.embed_dim, cfg.ffn_dim), (cfg.embed_dim, cfg.ffn_dim), (cfg.ffn_dim, cfg.embed_dim)]
    mats.append((cfg.embed_dim, cfg.vocab_size))

    def mat_bytes(k, n):
        if quant == "w8":
            return k * n + n * dtype_bytes
        if quant == "w4g128":
            return k * n // 2 + (k // 128) * n * dtype_bytes
        return k * n * dtype_bytes

    sb = 4 if f32_stream else dtype_bytes
    weights = sum(mat_bytes(k, n) for k, n in mats) + sb * (cfg.num_layers * 2 * cfg.embed_dim + cfg.embed_dim)
    kv_row = cfg.num_layers * 2 * cfg.num_kv_heads * cfg.head_dim
    return weights + dtype_bytes * (kv_row * (cache_len + 1) + cfg.embed_dim) + sb * cfg.vocab_size


def _ref_lib():
    """oracle/_ref: the reference C backend's kernels compiled from the reference checkout (test infrastructure)."""
    ref_dir = os.path.join(ROOT, "oracle", "_ref")
    flags = open("/proc/cpuinfo").read()
    name = "libgptrs_c_ref_avx512.so" if (" avx512f" in flags and " fma" in flags) else "libgptrs_c_ref_avx2.so"
    path = os.path.join(ref_dir, name)
    if not os.path.exists(path):
        return None, name
    lib = ctypes.CDLL(path)
    fp = ctypes.POINTER(ctypes.c_float)
    lib.gptrs_ref_cache_new.restype = ctypes.c_void_p
    lib.gptrs_ref_cache_free.argtypes = [ctypes.c_void_p]
    lib.gptrs_ref_matmul_f32_cached.argtypes = [fp, fp, fp, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p]
    return lib, name


def host_cores() -> int:
    """Worker processes for the all-cores figures: the cores this process may run on, capped by the share the
    environment grants (OMP_NUM_THREADS is set to it on the GPU box)."""
    n = len(os.sched_getaffinity(0))
    cap = os.environ.get("OMP_NUM_THREADS", "")
    if cap.isdigit() and int(cap) > 0:
        n = min(n, int(cap))
    return max(n, 1)


def _fork_all(n: int, work):
    """Runs work(i) -> float in n forked children at once (the parent's weights and packed caches are shared
    copy-on-write) and returns their results.  Only called before the process has touched the GPU."""
    pipes = []
    for i in range(n):
        r, w = os.pipe()
        pid = os.fork()
        if pid == 0:
            code = 0
            try:
                os.close(r)
                os.write(w, struct.pack("<d", float(work(i))))
            except BaseException:
                code = 1
            os._exit(code)
        os.close(w)
        pipes.append((pid, r))
    out = []
    for pid, r in pipes:
        data = os.read(r, 8)
        os.close(r)
        os.waitpid(pid, 0)
        out.append(struct.unpack("<d", data)[0] if len(data) == 8 else float("nan"))
    return out


def cpu_baseline(cfg, seconds_budget: float = 20.0):
    """Reference C kernels (gpt_rs_c_matmul_f32_cached_b, GEMV path, packed-B cache warm), f32 (the reference executes no
    bf16).  Sample: ONE layer's five weight matrices plus a 1/8 column slice of lm_head; a token = 26 layers + the full
    lm_head, extrapolated linearly.  One core (the C backend is single-threaded: the faithful figure), then the same
    loop in one process per core at once (independent sequences), with the core count stated."""
    lib, name = _ref_lib()
    if lib is None:
        return None
    fp = ctypes.POINTER(ctypes.c_float)
    a = cfg.attention_config()
    d = cfg.embed_dim
    head_cols = cfg.vocab_size // 8
    f = cfg.ffn_dim
    shapes = [(d, a.total_projection_dim), (a.query_projection_dim, d), (d, f), (d, f), (f, d), (d, head_cols)]
    nl = len(shapes) - 1
    rng = np.random.default_rng(0)
    mats, caches, xs, ys = [], [], [], []
    for k, n in shapes:
        w = rng.standard_normal((k, n), dtype=np.float32)
        w *= np.float32(0.02)
        mats.append(w)
        caches.append(lib.gptrs_ref_cache_new())
        xs.append(rng.standard_normal((1, k), dtype=np.float32))
        ys.append(np.empty((1, n), np.float32))

    def call(i):
        k, n = shapes[i]
        lib.gptrs_ref_matmul_f32_cached(xs[i].ctypes.data_as(fp), mats[i].ctypes.data_as(fp), ys[i].ctypes.data_as(fp), 1, n, k, caches[i])

    for i in range(len(shapes)):
        call(i)  # packs B once (gpt_rs_c_prepare warms this cache in the reference)

    def token_time(budget, max_reps):
        t_layer, t_head, reps = 0.0, 0.0, 0
        t_start = time.perf_counter()
        while reps < 2 or (time.perf_counter() - t_start < budget and reps < max_reps):
            t0 = time.perf_counter()
            for i in range(nl):
                call(i)
            t1 = time.perf_counter()
            call(nl)
            t2 = time.perf_counter()
            t_layer += t1 - t0
            t_head += t2 - t1
            reps += 1
        return cfg.num_layers * t_layer / reps + 8 * t_head / reps, reps

    t_token, reps = token_time(seconds_budget / 3, 20)
    cores = host_cores()
    all_cores = None
    if cores > 1:
        times = _fork_all(cores, lambda i: token_time(seconds_budget / 3, 20)[0])
        if all(t == t and t > 0 for t in times):
            all_cores = {"value": round(sum(1.0 / t for t in times), 3), "unit": "tokens/s", "cores": cores, "nproc": os.cpu_count(),
                         "how": "one process per core at once, each an independent sequence over the shared weights"}
    for c in caches:
        lib.gptrs_ref_cache_free(c)
    return {"value": round(1.0 / t_token, 4), "unit": "tokens/s", "cores": 1, "kind": "reference",
            "sample": f"{reps} reps of one layer's {nl} f32 GEMVs + 1/8 of lm_head through {name} "
                      f"(gpt_rs_c_matmul_f32_cached_b, m=1, packed-B cache warm); token time = {cfg.num_layers} layers + "
                      f"8 head slices; non-GEMV ops excluded", "all_cores": all_cores}


class _HostParams:
    """Backend stand-in that keeps materialised parameters on the host (weights for the CPU baseline come out of the
    same seeded initialiser the device model uses)."""

    def __init__(self):
        self.arrays = []

    def materialize(self, spec, data):
        self.arrays.append(np.frombuffer(bytes(data), "<f4").reshape(spec.dims).copy())
        return len(self.arrays) - 1

    def param_resolver(self):
        return self

    def set(self, sid, handle):
        pass


def cpu_gpt2_baseline(prompt, new_tokens: int, capacity: int = 128):
    """The CPU baseline workload: GPT-2 small f32 greedy decode with a KV cache on the reference C kernels
    (oracle/ref_harness.c: every matrix product through gpt_rs_c_matmul_f32_cached_b with a warm packed-B cache, the
    other ops as plain C loops), same seeded weights and prompt as the device run.  The prompt goes through token by
    token (the harness has no batched prefill); timed: the last `new_tokens` steps, steady decode.  One core, then one
    process per core at once."""
    lib, name = _ref_lib()
    if lib is None or not hasattr(lib, "gptrs_ref_gpt2_generate"):
        return None
    from gptrs_amd import models
    cfg = models.GptConfig()
    host = _HostParams()
    m = models.Gpt.random(cfg, host, seed=0, dtype="F32")
    P = dict(zip(m.param_names, host.arrays))
    L, d, f = cfg.num_layers, cfg.embed_dim, cfg.embed_dim * cfg.mlp_ratio
    fp = ctypes.POINTER(ctypes.c_float)
    fpp = ctypes.POINTER(fp)

    def ptr(a):
        return a.ctypes.data_as(fp)

    def per_layer(fmt):
        arr = (fp * L)(*[ptr(P[fmt.format(i)]) for i in range(L)])
        return arr

    class W(ctypes.Structure):
        _fields_ = [("tok_emb", fp), ("pos_emb", fp), ("ln1_g", fpp), ("ln1_b", fpp), ("w_qkv", fpp), ("b_qkv", fpp),
                    ("w_out", fpp), ("b_out", fpp), ("ln2_g", fpp), ("ln2_b", fpp), ("w_in", fpp), ("b_in", fpp),
                    ("w_o2", fpp), ("b_o2", fpp), ("lnf_g", fp), ("lnf_b", fp), ("lm_head", fp),
                    ("caches", ctypes.POINTER(ctypes.c_void_p)), ("layers", ctypes.c_int), ("d", ctypes.c_int),
                    ("heads", ctypes.c_int), ("f", ctypes.c_int), ("vocab", ctypes.c_int), ("capacity", ctypes.c_int),
                    ("eps", ctypes.c_float)]

    keep = [per_layer(x) for x in ("blocks.{}.ln_1.gamma", "blocks.{}.ln_1.beta", "blocks.{}.attention.w_qkv", "blocks.{}.attention.b_qkv",
                                   "blocks.{}.attention.w_out", "blocks.{}.attention.b_out", "blocks.{}.ln_2.gamma", "blocks.{}.ln_2.beta",
                                   "blocks.{}.feed_forward.w_in", "blocks.{}.feed_forward.b_in", "blocks.{}.feed_forward.w_out",
                                   "blocks.{}.feed_forward.b_out")]
    ncache = 4 * L + 1
    caches = (ctypes.c_void_p * ncache)(*[lib.gptrs_ref_cache_new() for _ in range(ncache)])
    w = W(ptr(P["tok_embeddings.weight"]), ptr(P["pos_embeddings"]), *[ctypes.cast(k, fpp) for k in keep],
          ptr(P["final_ln.gamma"]), ptr(P["final_ln.beta"]), ptr(P["lm_head"]), caches, L, d, cfg.num_heads, f, cfg.vocab_size,
          capacity, cfg.eps)
    lib.gptrs_ref_gpt2_generate.restype = ctypes.c_double
    lib.gptrs_ref_gpt2_generate.argtypes = [ctypes.POINTER(W), ctypes.POINTER(ctypes.c_int), ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                            fp, fp, fp, ctypes.POINTER(ctypes.c_int)]
    n_prompt = len(prompt)
    if n_prompt + new_tokens > capacity:
        return None
    prompt_arr = (ctypes.c_int * n_prompt)(*prompt)

    def run(n_new):
        kc = np.zeros(L * cfg.num_heads * capacity * (d // cfg.num_heads), np.float32)
        vc = np.zeros_like(kc)
        scratch = np.zeros(4 * d + 3 * d + f + capacity + cfg.vocab_size, np.float32)
        toks = (ctypes.c_int * n_new)()
        sec = lib.gptrs_ref_gpt2_generate(ctypes.byref(w), prompt_arr, n_prompt, n_new, n_new - 1, ptr(kc), ptr(vc), ptr(scratch), toks)
        return sec, list(toks)

    run(2)                       # packs every B once (the reference warms the caches in gpt_rs_c_prepare)
    sec, tokens = run(new_tokens)
    steps = new_tokens - 1
    cores = host_cores()
    all_cores = None
    if cores > 1:
        times = _fork_all(cores, lambda i: run(new_tokens)[0])
        if all(t == t and t > 0 for t in times):
            all_cores = {"value": round(sum(steps / t for t in times), 1), "unit": "tokens/s", "cores": cores, "nproc": os.cpu_count(),
                         "how": "one process per core at once, each generating the same sequence over the shared weights"}
    for c in caches:
        lib.gptrs_ref_cache_free(c)
    return {"value": round(steps / sec, 2), "unit": "tokens/s", "cores": 1, "kind": "reference",
            "sample": f"{steps} steady decode steps (cache length {n_prompt + 1}..{n_prompt + steps}) of GPT-2 small f32 through {name}: "
                      f"49 GEMVs per step via gpt_rs_c_matmul_f32_cached_b (packed-B caches warm), LayerNorm / bias / GELU / attention / "
                      f"argmax as plain C loops", "all_cores": all_cores, "tokens": tokens}


def microbench(args, be):
    """BASELINE configs[1]: single-op PTIR programs, f32 and bf16: dot_general [M,K]x[K,N] for M in {1, 8, 64, 512} and
    (K,N) in {(768,2304), (768,3072), (3072,768)}, softmax and layer_norm on [M,768]; plus the prefill GEMM shapes of
    the Ministral-3B layer at M = 1024 (bf16, SwiGLU pair as one dual GEMM).  Inputs N(0,1) from seed 2 (weights scaled
    by 1/sqrt(K)), resident on the device; each program runs `--steps` times after `--warmup`, wall clock with a device
    sync at both ends (cached plan, graph replay where the plan has enough steps)."""
    from gptrs_amd import functional as F
    from gptrs_amd.ptir import FunctionBuilder, Program, TensorSpec, f32_to_bf16_bits
    rng = np.random.default_rng(2)
    steps, warmup = (50, 5) if args.steps == 224 else (args.steps, max(args.warmup, 1))

    def upload(arr, dtype):
        data = arr.astype(np.float32).tobytes() if dtype == "F32" else f32_to_bf16_bits(arr.astype(np.float32)).tobytes()
        return be.materialize(TensorSpec(dtype, list(arr.shape)), data)

    def timed(prog, handles):
        for _ in range(warmup):
            be.run_program(prog, handles)
        be.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            be.run_program(prog, handles)
        be.synchronize()
        return (time.perf_counter() - t0) / steps

    results = []
    for dtype, es in (("F32", 4), ("Bf16", 2)):
        for k, n in ((768, 2304), (768, 3072), (3072, 768)):
            w = upload(rng.standard_normal((k, n), dtype=np.float32) / np.float32(np.sqrt(k)), dtype)
            for m in (1, 8, 64, 512):
                fb = FunctionBuilder("main", dtype)
                x, wp = fb.param(dtype, [m, k]), fb.param(dtype, [k, n])
                fb.set_results([x.matmul(wp)])
                dt = timed(Program(fb), [upload(rng.standard_normal((m, k), dtype=np.float32), dtype), w])
                nbytes, flops = (m * k + k * n + m * n) * es, 2.0 * m * k * n
                results.append({"op": "dot_general", "dtype": dtype, "m": m, "k": k, "n": n, "us": round(dt * 1e6, 2),
                                "gb_per_s": round(nbytes / dt / 1e9, 1), "tflop_per_s": round(flops / dt / 1e12, 3)})
        for m in (1, 8, 64, 512):
            for op in ("softmax", "layer_norm"):
                fb = FunctionBuilder("main", dtype)
                x = fb.param(dtype, [m, 768])
                hs = [upload(rng.standard_normal((m, 768), dtype=np.float32), dtype)]
                if op == "softmax":
                    fb.set_results([F.softmax_last_axis(x)])
                    nbytes = 2 * m * 768 * es
                else:
                    g, b = fb.param(dtype, [768]), fb.param(dtype, [768])
                    hs += [upload(rng.standard_normal(768, dtype=np.float32), dtype), upload(rng.standard_normal(768, dtype=np.float32), dtype)]
                    fb.set_results([F.layer_norm(x, g, b, 1e-5)[0]])
                    nbytes = (2 * m * 768 + 2 * 768) * es
                dt = timed(Program(fb), hs)
                results.append({"op": op, "dtype": dtype, "m": m, "n": 768, "us": round(dt * 1e6, 2), "gb_per_s": round(nbytes / dt / 1e9, 1)})
    m = 1024
    for k, n, dual in ((3072, 6144, False), (4096, 3072, False), (3072, 9216, True), (9216, 3072, False)):
        fb = FunctionBuilder("main", "Bf16")
        x, wp = fb.param("Bf16", [m, k]), fb.param("Bf16", [k, n])
        hs = [upload(rng.standard_normal((m, k), dtype=np.float32), "Bf16"),
              upload(rng.standard_normal((k, n), dtype=np.float32) / np.float32(np.sqrt(k)), "Bf16")]
        if dual:
            w2 = fb.param("Bf16", [k, n])
            hs.append(upload(rng.standard_normal((k, n), dtype=np.float32) / np.float32(np.sqrt(k)), "Bf16"))
            fb.set_results([F.swiglu(x.matmul(wp), x.matmul(w2))])
        else:
            fb.set_results([x.matmul(wp)])
        dt = timed(Program(fb), hs)
        flops = 2.0 * m * k * n * (2 if dual else 1)
        results.append({"op": "prefill_gemm" + ("_swiglu_pair" if dual else ""), "dtype": "Bf16", "m": m, "k": k, "n": n, "us": round(dt * 1e6, 2),
                        "tflop_per_s": round(flops / dt / 1e12, 1), "mfma_frac": round(flops / dt / 1e12 / MFMA_PEAK_TFLOPS, 4)})
    print(json.dumps({"metric": "single-op microbench (BASELINE configs[1]) + Ministral prefill GEMM shapes", "unit": "us per program run",
                      "n_gpus": 1, "steps": steps, "warmup": warmup, "data": "synthetic", "peaks": {"hbm_gb_per_s": HBM_PEAK_GBPS,
                      "bf16_mfma_tflop_per_s": MFMA_PEAK_TFLOPS}, "results": results}))


README_GPT2_TOKENS_PER_S = 74.71   # reference README.md:18-25: GPT-2 small f32, generate 64 tokens, C backend, 1 thread of a Ryzen 9 9950X3D


def chain_floor_record(be, phases: int = 157, reps: int = 20):
    """What a decode chain of `phases` phases costs when there is next to nothing to stream: a persistent launch over
    dependent bf16 linears alternating [1, 64] x [64, 3072] (every workgroup takes part: staging, one j-step, epilogue,
    barrier) and [1, 3072] x [3072, 64] (six workgroups work, all meet at the barrier), 393 KB of weights per phase.  The
    launch time (HIP events of the library's "profile" option around the launch) over the number of phases is the
    synchronisation cost per phase that a real chain pays on top of its streaming."""
    from gptrs_amd.ptir import FunctionBuilder, Program, f32_to_bf16_bits

    def build():
        fb = FunctionBuilder("main")
        h = fb.param("Bf16", [1, 64])
        for i in range(phases):
            h = h.matmul(fb.param("Bf16", [64, 3072] if i % 2 == 0 else [3072, 64]))
        fb.set_results([h])
        return Program(fb)

    prog = build()
    rng = np.random.default_rng(5)
    handles = []
    for spec in prog.param_specs:
        a = (rng.standard_normal(spec.dims) * 0.02).astype(np.float32)
        handles.append(be.materialize(spec, (f32_to_bf16_bits(a)).tobytes()))
    for _ in range(3):
        be.run_program(prog, handles, None)
    be.synchronize()
    c0, p0 = be.counter("chain_launches"), be.counter("chain_phases")
    be.set_option("profile", 1)
    for _ in range(reps):
        be.run_program(prog, handles, None)
    t_ns, calls = be.counter("linear_time_ns"), be.counter("linear_calls")
    be.set_option("profile", 0)
    chains, ph = be.counter("chain_launches") - c0, be.counter("chain_phases") - p0
    if chains != reps or calls != reps or ph != reps * phases:
        return {"error": "the probe program did not run as one chain launch per call", "chains": chains, "calls": calls, "phases": ph}
    us = t_ns / calls / 1e3
    return {"phases": phases, "us_per_launch": round(us, 1), "us_per_phase": round(us / phases, 2),
            "what": "persistent launch over %d dependent bf16 linears with 393 KB of weights each (alternating 64 -> 3072 and 3072 -> 64): "
                    "grid barrier, staging, one or three j-steps, epilogue and store acknowledgement per phase, nothing to stream" % phases}


def quant_record(be, cfg, quant: str, prompt, capacity: int, steps: int = 64, warmup: int = 8, prof_steps: int = 16):
    """The headline workload with weight-only quantised linears (BASELINE configs[4]; every linear incl. lm_head as int8
    per output channel or int4 groups of 128, activations / KV cache / embeddings bf16, f32 residual stream): steady
    decode rate, and the persistent launch priced with the step's algorithmic bytes (codes + scales once, valid KV
    once), timed with HIP events on the backend's stream."""
    from gptrs_amd import models
    t0 = time.perf_counter()
    model = models.Ministral.random(cfg, be, seed=5, dtype="Bf16", quant=quant, residual_dtype="F32")
    t_init = time.perf_counter() - t0
    gen = models.Generator(model, prompt, kv_cache_capacity=capacity)
    for _ in range(warmup):
        gen.step()
    be.synchronize()
    start = gen.processed_len
    t0 = time.perf_counter()
    for _ in range(steps):
        gen.step()
    be.synchronize()
    t_step = (time.perf_counter() - t0) / steps
    launches = be.counter("last_program_launches")
    step_bytes = algorithmic_bytes_per_step(cfg, 2, start + steps // 2, quant, True)
    prof_start = gen.processed_len
    c0, p0 = be.counter("chain_launches"), be.counter("chain_phases")
    be.set_option("profile", 1)
    for _ in range(prof_steps):
        gen.step()
    t_ns, calls = be.counter("linear_time_ns"), be.counter("linear_calls")
    be.set_option("profile", 0)
    chains, phases = be.counter("chain_launches") - c0, be.counter("chain_phases") - p0
    roof = None
    if t_ns > 0 and chains == calls and calls > 0:
        nbytes = sum(algorithmic_bytes_per_step(cfg, 2, prof_start + i, quant, True) for i in range(prof_steps))
        achieved = nbytes / (t_ns * 1e-9) / 1e9
        roof = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": chain_traffic_bytes("w8_bytes") if quant == "w8" and cfg.num_layers == 26 and len(prompt) == 1024 else None,
                "kernel": "chain_kernel over %s code words, %d phases per launch" % (quant, phases // max(chains, 1)),
                "launches": calls, "avg_launch_us": round(t_ns / calls / 1e3, 2), "bytes_per_launch": round(nbytes / calls)}
    return {"metric": "decode tokens/s, Ministral-3B-shape %s weight-only linears (lm_head included), batch 1" % quant,
            "value": round(1.0 / t_step, 2), "unit": "tokens/s", "steps": steps, "warmup": warmup, "ms_per_step": round(t_step * 1e3, 4),
            "dtype": "bf16 activations, %s weights" % ("int8" if quant == "w8" else "int4"), "data": "synthetic",
            "hbm_gbps": round(step_bytes / t_step / 1e9, 1), "hbm_frac": round(step_bytes / t_step / 1e9 / HBM_PEAK_GBPS, 4),
            "algorithmic_bytes_per_step": step_bytes, "launches_per_step": launches, "weight_init_s": round(t_init, 1), "roofline": roof}


def gpt2_record(be, steps: int, warmup: int, cpu=None):
    """BASELINE configs[0]: GPT-2 small f32, weights N(0, 0.02) from seed 0, prompt of 16 ids (seed 1), greedy, 64 tokens
    with KV cache (capacity 128).  Timed like the reference's published figure (README.md:27-50,
    scripts/gptrs_eval/runner.py:24-56): each step is one WHOLE generate call, prefill included; tokens/s = 64 / mean
    wall time.  The steady decode rate and its share of the HBM roofline are reported beside it."""
    from gptrs_amd import models
    cfg = models.GptConfig()
    t0 = time.perf_counter()
    model = models.Gpt.random(cfg, be, seed=0, dtype="F32")
    t_init = time.perf_counter() - t0
    prompt = np.random.default_rng(1).integers(0, cfg.vocab_size, 16).tolist()
    new_tokens = 64

    def generate():
        gen = models.Generator(model, prompt, kv_cache_capacity=128)
        out = gen.generate(new_tokens)
        be.synchronize()
        return out

    for _ in range(max(warmup, 1)):
        tokens = generate()
    t0 = time.perf_counter()
    for _ in range(steps):
        assert generate() == tokens
    elapsed = (time.perf_counter() - t0) / steps
    gen = models.Generator(model, prompt, kv_cache_capacity=256)
    for _ in range(8):
        gen.step()
    be.synchronize()
    n, start = 128, gen.processed_len
    t0 = time.perf_counter()
    for _ in range(n):
        gen.step()
    be.synchronize()
    t_step = (time.perf_counter() - t0) / n
    d, L, V = cfg.embed_dim, cfg.num_layers, cfg.vocab_size
    per_layer = d * 3 * d + d * d + 2 * d * cfg.mlp_ratio * d + (3 * d + d + cfg.mlp_ratio * d + d) + 4 * d   # weights, biases, LN
    step_bytes = 4 * (L * per_layer + 2 * d + d * V + 2 * L * d * (start + n // 2 + 1) + V + 2 * d)
    value = new_tokens / elapsed
    if cpu is not None:
        cpu = dict(cpu)
        cpu["same_tokens_as_device"] = cpu.pop("tokens", None) == tokens
    return {
        "metric": "tokens/s of a whole generate call (prefill 16 + 64 greedy tokens), GPT-2 small f32, batch 1",
        "value": round(value, 2), "unit": "tokens/s", "steps": steps, "warmup": max(warmup, 1),
        "ms_per_step": round(elapsed * 1e3, 4),
        "vs_baseline": round(value / README_GPT2_TOKENS_PER_S, 2), "dtype": "f32", "data": "synthetic",
        "config": {"workload": "gpt-2 small f32, prompt 16, greedy generate 64 with KV cache (capacity 128); a step is one generate call",
                   "baseline": "74.71 tokens/s: reference C backend, one thread of a Ryzen 9 9950X3D, 1-token prompt, sampled (README.md:18-25)"},
        "decode_steady_tokens_per_s": round(1.0 / t_step, 1), "decode_us_per_step": round(t_step * 1e6, 1),
        "hbm_gbps": round(step_bytes / t_step / 1e9, 1), "hbm_frac": round(step_bytes / t_step / 1e9 / HBM_PEAK_GBPS, 4),
        "algorithmic_bytes_per_step": step_bytes, "launches_per_step": be.counter("last_program_launches"),
        "chain_launches_per_step": None,
        "weight_init_s": round(t_init, 1), "cpu_baseline": cpu}


def batched_decode(args, be, cfg, model, capacity):
    """B independent sequences decoded together (models.BatchGenerator): tokens/s summed over the sequences.  The next
    tokens are the row-wise argmax taken on the device and fed to the next step there (4 B bytes reach the host per
    step), the linear layers are bracketed by HIP events in a second pass as in the batch-1 run."""
    B = args.batch
    from gptrs_amd import models
    rng = np.random.default_rng(6)
    rows = [rng.integers(0, cfg.vocab_size, args.prompt).tolist() for _ in range(B)]
    gen = models.BatchGenerator(model, rows, kv_cache_capacity=capacity)   # first call compiles the plan
    be.synchronize()
    times = []
    for _ in range(3):   # median of three timed prefills
        del gen
        t0 = time.perf_counter()
        gen = models.BatchGenerator(model, rows, kv_cache_capacity=capacity)
        be.synchronize()
        times.append(time.perf_counter() - t0)
    t_prefill = sorted(times)[1]
    state = {"pos": args.prompt}

    def step():
        gen.step()
        state["pos"] += 1

    for _ in range(args.warmup):
        step()
    be.synchronize()
    start_len = state["pos"]
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    be.synchronize()
    elapsed = time.perf_counter() - t0
    launches = be.counter("last_program_launches")
    prof_steps = min(8, capacity - state["pos"] - 1)
    roof = None
    if prof_steps > 0:
        be.set_option("profile", 1)
        for _ in range(prof_steps):
            step()
        t_ns, calls, nbytes = be.counter("linear_time_ns"), be.counter("linear_calls"), be.counter("linear_bytes")
        be.set_option("profile", 0)
        if t_ns > 0:
            achieved = nbytes / (t_ns * 1e-9) / 1e9
            roof = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                    "kernel": "skinny_gemm_kernel: all linear layers of a batched decode step (weights once, %d activation rows)" % B,
                    "launches": calls, "avg_launch_us": round(t_ns / max(calls, 1) / 1e3, 2),
                    "bytes_per_launch": round(nbytes / max(calls, 1))}
    wname = {"none": "bf16", "w8": "int8-weight-only (per output channel) bf16", "w4g128": "int4-weight-only (groups of 128) bf16"}[args.quant]
    mid_len = start_len + args.steps // 2
    kv_bytes = 2 * cfg.num_layers * cfg.num_kv_heads * cfg.head_dim * 2 * (mid_len + 1)
    step_bytes = algorithmic_bytes_per_step(cfg, 2, mid_len, args.quant, args.residual == "f32") + (B - 1) * kv_bytes   # weights once, every sequence's KV
    print(json.dumps({
        "metric": "decode tokens/s summed over %d sequences, Ministral-3B-shape %s (side workload: batched decode)" % (B, wname),
        "value": round(B * args.steps / elapsed, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "ministral-3b-shape %s decode, batch %d, prompt %d each, greedy, KV capacity %d" % (wname, B, args.prompt, capacity),
                   "layers": cfg.num_layers, "cache_len_mid": mid_len},
        "hbm_gbps": round(step_bytes / (elapsed / args.steps) / 1e9, 1),
        "hbm_frac": round(step_bytes / (elapsed / args.steps) / 1e9 / HBM_PEAK_GBPS, 4),
        "algorithmic_bytes_per_step": step_bytes, "launches_per_step": launches,
        "prefill_ms": round(t_prefill * 1e3, 2), "prefill_tokens": B * args.prompt, "roofline": roof, "cpu_baseline": None}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=224)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--prompt", type=int, default=1024)
    ap.add_argument("--layers", type=int, default=26, help="debug only: fewer layers is NOT the benchmark config")
    ap.add_argument("--quant", choices=["none", "w8", "w4g128"], default="none",
                    help="weight-only quantisation of every linear weight (BASELINE configs[4]: w8 = int8 per output channel, "
                         "w4g128 = int4 in groups of 128); activations, KV cache and embeddings stay bf16")
    ap.add_argument("--batch", type=int, default=1,
                    help="B > 1: batched decode of B independent sequences (rows stacked through the linear layers, one attention "
                         "launch per layer for all of them); a side workload, NOT the headline metric (which is batch 1)")
    ap.add_argument("--model", choices=["ministral", "gpt2"], default="ministral",
                    help="gpt2: the reference's own published workload (GPT-2 small f32, generate 64 tokens); --steps then counts "
                         "whole generate calls (default 8)")
    ap.add_argument("--microbench", action="store_true",
                    help="single-op programs of BASELINE configs[1] (dot_general / softmax / layer_norm, f32 and bf16) and the "
                         "Ministral prefill GEMM shapes; prints one JSON line with a result per shape")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--residual", choices=["f32", "bf16"], default="f32",
                    help="f32 (default): bf16 weights and matmul operands with an f32 residual stream, f32 norms and f32 logits "
                         "(DotGeneral out_dtype); bf16: every tensor of the program is bf16")
    ap.add_argument("--no-front-end", action="store_true",
                    help="hand the backend the emitters' instruction stream; default: every model program goes through the "
                         "reference's optimizer pipeline first (gpt.rs_amd/front_end.py), as the reference's arena does")
    ap.add_argument("--no-gpt2", action="store_true", help="skip the GPT-2 small f32 sub-record of the default run")
    ap.add_argument("--no-int8", action="store_true", help="skip the int8 weight-only sub-record (BASELINE configs[4]) of the default run")
    ap.add_argument("--no-floor", action="store_true", help="skip the chain_floor sub-record (a chain with nothing to stream) of the default run")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain elementwise kernel of known traffic (x + 0 over 2^28 f32: 1 GiB read, 1 GiB written, "
                         "kernel binary_scalar_kernel) so FETCH_SIZE / WRITE_SIZE can be scaled to bytes")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no sharding); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    entry.load_package()
    from gptrs_amd import models
    from gptrs_amd.backend import HipBackend

    # CPU baselines first: they fork one worker per core, which must happen before this process touches the GPU
    plain_run = not (args.copy_calibration or args.microbench)
    cpu_main = cpu_gpt2 = None
    if plain_run and not args.no_cpu_baseline:
        if args.model == "gpt2" or (args.batch == 1 and not args.no_gpt2):
            cpu_gpt2 = cpu_gpt2_baseline(np.random.default_rng(1).integers(0, models.GptConfig().vocab_size, 16).tolist(), 64)
        if args.model == "ministral" and args.batch == 1:
            cpu_main = cpu_baseline(models.MinistralConfig(num_layers=args.layers))

    be = HipBackend(0)
    if args.copy_calibration:
        from gptrs_amd.ptir import FunctionBuilder, Program, TensorSpec
        n = 1 << 28
        fb = FunctionBuilder("main")
        x = fb.param("F32", [n])
        fb.set_results([x + 0.0])
        prog = Program(fb)
        h = be.materialize(TensorSpec("F32", [n]), None)
        for _ in range(10):
            be.run_program(prog, [h])
        be.synchronize()
        print(json.dumps({"copy_calibration": "10 launches of x + 0.0 over %d f32" % n, "bytes_read_per_launch": 4 * n, "bytes_written_per_launch": 4 * n}))
        return
    if args.microbench:
        return microbench(args, be)
    if args.model == "gpt2":
        if args.steps == 224:
            args.steps, args.warmup = 8, 2
        rec = gpt2_record(be, args.steps, args.warmup, cpu_gpt2)
        rec.update({"n_gpus": 1, "higher_is_better": True, "scaling": "weak", "roofline": None})
        print(json.dumps(rec))
        return
    cfg = models.MinistralConfig(num_layers=args.layers)
    f32_stream = args.residual == "f32"
    total_len = args.prompt + args.warmup + args.steps + 1
    capacity = max(1280, (total_len + 255) // 256 * 256)
    if capacity > cfg.context_length:
        raise SystemExit(f"prompt + warmup + steps = {total_len} exceeds the context length {cfg.context_length}")
    t0 = time.perf_counter()
    model = models.Ministral.random(cfg, be, seed=5, dtype="Bf16", quant=None if args.quant == "none" else args.quant,
                                    residual_dtype="F32" if f32_stream else None)
    t_init = time.perf_counter() - t0
    model.front_end = not args.no_front_end
    prompt = np.random.default_rng(6).integers(0, cfg.vocab_size, args.prompt).tolist()
    if args.batch > 1:
        return batched_decode(args, be, cfg, model, capacity)

    # prefill (reported separately, crates/gpt-rs-cli/src/main.rs:900-935): first call compiles the plan
    gen = models.Generator(model, prompt, kv_cache_capacity=capacity)
    be.synchronize()
    times = []
    for _ in range(3):   # median of three timed prefills
        t0 = time.perf_counter()
        gen = models.Generator(model, prompt, kv_cache_capacity=capacity)
        be.synchronize()
        times.append(time.perf_counter() - t0)
    t_prefill = sorted(times)[1]

    for _ in range(args.warmup):
        gen.step()
    be.synchronize()
    start_len = gen.processed_len
    t0 = time.perf_counter()
    for _ in range(args.steps):
        gen.step()
    be.synchronize()
    elapsed = time.perf_counter() - t0
    launches = be.counter("last_program_launches")

    # second pass over fresh steps with the dominant launches bracketed by HIP events on the backend's
    # stream: the persistent decode chain (one launch per step carrying every linear layer and the
    # decode attention), or the per-linear GEMV kernels when the chain is switched off
    prof_steps = min(32, capacity - gen.processed_len - 1)
    roof = None
    if prof_steps > 0:
        prof_start = gen.processed_len
        chains0, phases0 = be.counter("chain_launches"), be.counter("chain_phases")
        be.set_option("profile", 1)
        for _ in range(prof_steps):
            gen.step()
        t_ns = be.counter("linear_time_ns")
        calls = be.counter("linear_calls")
        nbytes = be.counter("linear_bytes")
        be.set_option("profile", 0)
        chains = be.counter("chain_launches") - chains0
        if t_ns > 0:
            if chains == calls:
                # the timed launches are whole decode steps minus embedding and argmax: price them with
                # the step's algorithmic bytes (weights once, valid KV once, logits once)
                nbytes = sum(algorithmic_bytes_per_step(cfg, 2, prof_start + i, args.quant, f32_stream) for i in range(prof_steps))
                kernel = "chain_kernel: persistent decode chain, %d phases per launch (all linear layers + decode attention of a step)" % (
                    (be.counter("chain_phases") - phases0) // max(chains, 1))
            else:
                kernel = "gemv_tiled_kernel<bf16>: all linear layers of a decode step"
            achieved = nbytes / (t_ns * 1e-9) / 1e9
            default_workload = chains == calls and args.layers == 26 and args.prompt == 1024 and args.quant == "none"
            roof = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBPS, 4),
                    "traffic": chain_traffic_bytes() if default_workload else None,
                    "kernel": kernel,
                    "launches": calls, "avg_launch_us": round(t_ns / max(calls, 1) / 1e3, 2),
                    "bytes_per_launch": round(nbytes / max(calls, 1))}

    mid_len = start_len + args.steps // 2
    step_bytes = algorithmic_bytes_per_step(cfg, 2, mid_len, args.quant, f32_stream)
    wname = {"none": "bf16", "w8": "int8-weight-only (per output channel) bf16", "w4g128": "int4-weight-only (groups of 128) bf16"}[args.quant]
    if f32_stream:
        wname += " (f32 residual stream and logits)"
    ms_per_step = elapsed / args.steps * 1e3
    # prefill against the matrix-core peak: the linear layers over every prompt row, causal attention (half of the
    # T x T products), the head on the last row
    a_ = cfg.attention_config()
    lin = cfg.embed_dim * a_.total_projection_dim + a_.query_projection_dim * cfg.embed_dim + 3 * cfg.embed_dim * cfg.ffn_dim
    prefill_flops = cfg.num_layers * (2.0 * args.prompt * lin + 4.0 * cfg.num_heads * args.prompt * args.prompt * cfg.head_dim / 2) + \
        2.0 * cfg.embed_dim * cfg.vocab_size
    prefill = {"ms": round(t_prefill * 1e3, 2), "tokens": args.prompt, "tflop": round(prefill_flops / 1e12, 3),
               "tflop_per_s": round(prefill_flops / t_prefill / 1e12, 1),
               "mfma_frac": round(prefill_flops / t_prefill / 1e12 / MFMA_PEAK_TFLOPS, 4), "peak_tflop_per_s": MFMA_PEAK_TFLOPS,
               "what": "wall time of one 1024-token prefill call (median of three; head on the last row), all launches included"}
    bytes_allocated = be.counter("bytes_allocated")
    gpt2 = int8 = None
    floor = chain_floor_record(be) if args.quant == "none" and not args.no_floor else None
    default_line = args.quant == "none" and args.layers == 26
    if default_line and not args.no_int8:
        del gen, model
        gen = model = None
        be.set_option("drop_derived_weights", 1)
        int8 = quant_record(be, cfg, "w8", prompt, capacity)
        be.set_option("drop_derived_weights", 1)
    if not args.no_gpt2:
        del gen, model
        gpt2 = gpt2_record(be, 8, 2, cpu_gpt2)
    out = {
        "metric": "decode tokens/s, Ministral-3B-shape %s batch 1 (HBM GB/s as %% of 8 TB/s in hbm_frac)" % wname,
        "value": round(args.steps / elapsed, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "ministral-3b-shape %s decode, batch 1, prompt %d, greedy, KV capacity %d" % (wname, args.prompt, capacity),
                   "layers": cfg.num_layers, "d_model": cfg.embed_dim, "heads": cfg.num_heads, "kv_heads": cfg.num_kv_heads,
                   "head_dim": cfg.head_dim, "ffn": cfg.ffn_dim, "vocab": cfg.vocab_size, "cache_len_mid": mid_len,
                   "program_stream": "emitters" if args.no_front_end else "optimizer pipeline (canonicalise, parameter-only fold, CSE, DCE) ahead of run_program"},
        "hbm_gbps": round(step_bytes / (elapsed / args.steps) / 1e9, 1),
        "hbm_frac": round(step_bytes / (elapsed / args.steps) / 1e9 / HBM_PEAK_GBPS, 4),
        "algorithmic_bytes_per_step": step_bytes,
        "launches_per_step": launches,
        "prefill_ms": round(t_prefill * 1e3, 2), "prefill_tokens": args.prompt,
        "weight_init_s": round(t_init, 1), "device_bytes_allocated": bytes_allocated,
        "roofline": roof,
        "cpu_baseline": cpu_main,
        "prefill": prefill,
        "chain_floor": floor,
        "int8": int8,
        "gpt2_f32": gpt2,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
