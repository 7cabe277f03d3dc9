#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

A step is one pass of the attention operator over one batch of synthetic input that is
already resident in HBM.  Workloads are the five configurations the metric is quoted on:

    prefill2   causal GQA prefill, T=2048, 40/8 heads, d=128            (MFMA bound)
    decode1    contiguous decode, 32/8 heads, d=128, context 4096        (HBM bound)
    paged3     32 sessions, paged bf16 KV, contexts U[512,16384]         (HBM bound)
    paged4     32 sessions, paged Q8_0 KV, contexts U[4096,32768]        (HBM bound)
    mla5       absorbed MLA decode, batch 16, 128 heads, context 8192    (HBM bound)

By name only (not configurations of the metric): exact2 and exact1 (configurations 2 and 1
under the EXACT_F32 contract: fp32 matrix cores, and double-precision split decode),
append_bf16 / append_q8_0 (the KV page writer), history_append (the token-major writer), paged3_p64 / paged4_p64
(configurations 3 and 4 with pages of 64 tokens), prefill_d256 / prefill_d64 (causal prefill at head
dimension 256, 24/4 heads, and 64, 16/4 heads), paged_d256 / paged_d64 and decode_d256 / decode_d64 (configurations 3 and 1
at those head dimensions), exact2_d256 / exact1_d256 (the EXACT_F32 forms at 24/4 heads, head dimension 256), decoder_block / decoder_block_fused (one decode step of the reference's decoder attention
block: call for call through the reference's slots, and through the two fused entry points), copy.

Prints ONE JSON line.  `value` is the headline workload's throughput; every workload
that ran is listed under "workloads" with its own roofline figures.  Timing uses HIP
events recorded on the backend's own stream (the stream the kernels are launched on).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from clori_amd import binding as B  # noqa: E402
from clori_amd.backend import Backend, kv_pack_pages, q8_0_encode_rows  # noqa: E402

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
MFMA_F32_PEAK_TFLOPS = 157.3    # MI355X dense fp32 matrix, published


def bf16_bits(x):
    """float32 -> bf16 bits (RNE) with integer arithmetic; inputs are finite."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_decode(bits):
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def random_bf16(rng, count, unique=1 << 24):
    """`count` N(0,1) bf16 values.  Beyond `unique` values the block repeats: throughput
    does not depend on the values and generation stays in seconds."""
    base = bf16_bits(rng.standard_normal(min(count, unique), dtype=np.float32))
    if count <= unique:
        return base
    reps = (count + unique - 1) // unique
    return np.tile(base, reps)[:count]


SPIN_UP_SECONDS = 0.2        # untimed work before the warm-up steps (--spin-up)


RECORD_ITERATIONS = 100       # per-dispatch samples of the benchmark record


def time_steps(backend, run, steps, warmup, kernels):
    """W untimed steps, then K steps bracketed by device events and by a synchronise on both
    sides: that is the step time `value` is computed from.  Afterwards, outside the timed
    region: for each kernel of the step, the same steps again with an event pair around
    every launch of that kernel (mean duration per launch, the first kernel named is the
    dominant one), and RECORD_ITERATIONS single dispatches each timed on the host and on the
    device, from which the benchmark record's distributions are taken."""
    from clori_amd.backend import benchmark_summarize
    backend.set_completion_mode(B.COMPLETION_DEFERRED)
    step = run
    # the part raises its clocks only under sustained load: keep it busy for SPIN_UP_SECONDS
    # before the W warm-up steps, all untimed
    spin_until = time.perf_counter() + SPIN_UP_SECONDS
    while time.perf_counter() < spin_until:
        for _ in range(16):
            step()
        backend.sync()
    for _ in range(warmup):
        step()
    backend.sync()
    t0 = time.perf_counter()
    backend.timing_begin()
    for _ in range(steps):
        step()
    device_ms = backend.timing_end()
    backend.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    kernel_ms = {}
    for kernel in kernels:
        backend.kernel_probe_begin(kernel)
        for _ in range(min(steps, 128)):
            run()
        launches, total_ms = backend.kernel_probe_end()
        backend.sync()
        if launches:
            kernel_ms[kernel] = total_ms / launches
    # per-dispatch samples: each dispatch completes (status read back) before the next starts
    backend.set_completion_mode(B.COMPLETION_IMMEDIATE)
    before = backend.memory_stats()
    host_s, device_s, facts = [], [], None
    for _ in range(RECORD_ITERATIONS):
        h0 = time.perf_counter()
        backend.timing_begin()
        facts = run()
        device_s.append(backend.timing_end() * 1e-3)
        host_s.append(time.perf_counter() - h0)
    after = backend.memory_stats()
    record = {"benchmark_scope": "attention_component", "warmup_count": warmup,
              "iteration_count": RECORD_ITERATIONS, "first_execution_ns": int(host_s[0] * 1e9 + 0.5)}
    record.update(benchmark_summarize(host_s))
    record["device_timing_available"] = True
    record.update(benchmark_summarize(device_s, prefix="device_"))
    record.update({
        "h2d_bytes": int(after.h2d_bytes - before.h2d_bytes),
        "d2h_bytes": int(after.d2h_bytes - before.d2h_bytes),
        "warm_device_allocations": int(after.allocation_events - before.allocation_events),
        "warm_device_frees": int(after.release_events - before.release_events),
        "last_dispatch_kernel_launches": int(facts.kernel_launches),
        "last_dispatch_peak_device_bytes": int(after.peak_allocated_bytes),
        "resident_bytes": int(after.allocated_bytes)})
    return dict(ms=device_ms / steps, wall_ms=wall_ms / steps, kernel_ms=kernel_ms, record=record)


# --------------------------------------------------------------------- workloads --

def decode_kernels(kernel, facts, finish="yvex_rocm_decode_finish"):
    """Kernels of one decode step.  A launch that does not fill the device merges its split
    segments in the kernel itself (one launch, the `_merged` build of the kernel); a full-size
    launch leaves the merge to a second, small kernel."""
    if facts.kernel_launches == 1:
        return [kernel + "_merged"]
    return [kernel, finish]


def workload_paged(backend, rng, steps, warmup, q8=False, page=16, hq=32, hkv=8, d=128, name=None):
    sessions = 32
    lo, hi = (4096, 32768) if q8 else (512, 16384)
    contexts = rng.integers(lo, hi + 1, size=sessions).astype(np.int32)
    need = (contexts + page - 1) // page
    pool_pages = int(need.sum())
    stride = int(hi // page)
    perm = rng.permutation(pool_pages).astype(np.int32)
    table = np.zeros((sessions, stride), dtype=np.int32)
    at = 0
    for s in range(sessions):
        table[s, :need[s]] = perm[at:at + need[s]]
        at += int(need[s])
    storage = B.KV_Q8_0 if q8 else B.KV_BF16
    block = 2176 if q8 else 32 * d           # one 16-token block; a page is page // 16 of them
    blocks = pool_pages * hkv * (page // 16)
    pool_bytes = blocks * block
    if q8:
        # N(0,1) values rounded to bf16 and quantised on the host with the library's Q8_0 encoder
        # (round-to-nearest absmax/127), packed into the device page layout.  A sample of
        # SAMPLE_PAGES pages is generated and repeated through the pool: throughput does not
        # depend on the values and generation stays in seconds.
        sample_pages = min(pool_pages, 2048)

        def quantised_pool(is_value):
            values = bf16_decode(random_bf16(rng, sample_pages * page * hkv * d))
            blocks = q8_0_encode_rows(values.reshape(sample_pages, page, hkv, d))
            packed = kv_pack_pages(blocks, B.KV_Q8_0, is_value, hkv, d, page)
            reps = (pool_bytes + packed.size - 1) // packed.size
            return np.tile(packed, reps)[:pool_bytes]
        k_pool = backend.tensor("k-pages", B.DTYPE_I8, (pool_bytes,), quantised_pool(False))
        v_pool = backend.tensor("v-pages", B.DTYPE_I8, (pool_bytes,), quantised_pool(True))
    else:
        k_pool = backend.tensor("k-pages", B.DTYPE_BF16, (pool_bytes // 2,),
                                random_bf16(rng, pool_bytes // 2))
        v_pool = backend.tensor("v-pages", B.DTYPE_BF16, (pool_bytes // 2,),
                                random_bf16(rng, pool_bytes // 2))
    q = backend.tensor("q", B.DTYPE_BF16, (sessions, hq, d), random_bf16(rng, sessions * hq * d))
    tt = backend.tensor("table", B.DTYPE_I32, table.shape, table)
    tc = backend.tensor("ctx", B.DTYPE_I32, contexts.shape, contexts)
    out = backend.tensor("out", B.DTYPE_BF16, (sessions, hq, d))
    lse = backend.tensor("lse", B.DTYPE_F32, (sessions, hq))
    req = backend.paged_requirement(sessions, hq, hkv, d, page, pool_pages, stride, hi,
                                    storage=storage)
    work = backend.tensor("workspace", B.DTYPE_I8,
                          (backend.paged_decode_workspace_required(req),))
    backend.workspace_attach(work)
    run = lambda: backend.paged_decode_execute(req, q, k_pool, v_pool, tt, tc, out, lse)  # noqa: E731
    facts = run()
    kernel = "yvex_rocm_decode_paged_q8_0" if q8 else \
        "yvex_rocm_decode_paged_bf16" + ("" if d == 128 else "_%d" % d)
    kernels = decode_kernels(kernel, facts, "yvex_rocm_decode_finish" + ("_256" if d == 256 else ""))
    timed = time_steps(backend, run, steps, warmup, kernels)
    backend.workspace_detach()
    tokens = int(contexts.sum())
    per_token = 2 * hkv * (136 if q8 else 2 * d)
    algo = tokens * per_token + int(need.sum()) * 4 + sessions * 4 + 2 * sessions * hq * d * 2 + \
        sessions * hq * 4
    assert np.all(np.isfinite(lse.read()))
    return dict(name=name or ("paged4" if q8 else "paged3") + ("" if page == 16 else "_p%d" % page),
                workload="paged %s GQA decode: 32 sessions, %d/%d heads, d=%d, contexts U[%d,%d], "
                         "%d-token pages, seeded permutation page tables%s" %
                         ("Q8_0" if q8 else "bf16", hq, hkv, d, lo, hi, page,
                          ", N(0,1) bf16 values quantised on the host (absmax/127, round to nearest), "
                          "a 2048-page sample repeated through the pool" if q8 else ""),
                bound="hbm", algorithmic_bytes=algo, tokens=tokens,
                launches=int(facts.kernel_launches), kernels=kernels, **timed)


def workload_decode1(backend, rng, steps, warmup, hq=32, hkv=8, d=128, name="decode1"):
    ctx = 4096
    q = backend.tensor("q", B.DTYPE_BF16, (1, hq, d), random_bf16(rng, hq * d))
    k = backend.tensor("k", B.DTYPE_BF16, (ctx, hkv, d), random_bf16(rng, ctx * hkv * d))
    v = backend.tensor("v", B.DTYPE_BF16, (ctx, hkv, d), random_bf16(rng, ctx * hkv * d))
    out = backend.tensor("out", B.DTYPE_BF16, (1, hq, d))
    lse = backend.tensor("lse", B.DTYPE_F32, (1, hq))
    req = backend.attention_requirement(1, ctx, hq, hkv, d, causal=True, query_start=ctx - 1,
                                        dtype=B.DTYPE_BF16,
                                        contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    work = backend.tensor("workspace", B.DTYPE_I8, (backend.attention_workspace_required(req),))
    backend.workspace_attach(work)
    run = lambda: backend.attention_execute(req, q, k, v, out, lse=lse)  # noqa: E731
    facts = run()
    # one launch: teams of eight waves (four at head dimension 256) per stretch of the history,
    # merged through LDS and then between the teams by the one that arrives last
    kernels = ["yvex_rocm_decode_rows_bf16_team" + ("" if d == 128 else "_%d" % d)]
    timed = time_steps(backend, run, steps, warmup, kernels)
    backend.workspace_detach()
    algo = 2 * ctx * hkv * d * 2 + 2 * hq * d * 2 + hq * 4
    return dict(name=name,
                workload="GQA decode: batch 1, %d/%d heads, d=%d, context 4096, contiguous bf16 KV" % (hq, hkv, d),
                bound="hbm", algorithmic_bytes=algo, tokens=ctx,
                launches=int(facts.kernel_launches), kernels=kernels, **timed)


def workload_prefill2(backend, rng, steps, warmup, hq=40, hkv=8, d=128, name="prefill2"):
    t = 2048
    sq = rng.uniform(0.5, 1.5, size=(1, hq, 1)).astype(np.float32)
    skv = rng.uniform(0.5, 1.5, size=(1, hkv, 1)).astype(np.float32)
    qv = bf16_bits(rng.standard_normal((t, hq, d), dtype=np.float32) * sq)
    kv = bf16_bits(rng.standard_normal((t, hkv, d), dtype=np.float32) * skv)
    vv = bf16_bits(rng.standard_normal((t, hkv, d), dtype=np.float32) * skv)
    q = backend.tensor("q", B.DTYPE_BF16, (t, hq, d), qv)
    k = backend.tensor("k", B.DTYPE_BF16, (t, hkv, d), kv)
    v = backend.tensor("v", B.DTYPE_BF16, (t, hkv, d), vv)
    out = backend.tensor("out", B.DTYPE_BF16, (t, hq, d))
    req = backend.attention_requirement(t, t, hq, hkv, d, causal=True, dtype=B.DTYPE_BF16,
                                        contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    run = lambda: backend.attention_execute(req, q, k, v, out)  # noqa: E731
    facts = run()
    kernels = ["yvex_rocm_prefill_bf16" + ("" if d == 128 else "_%d" % d)]
    timed = time_steps(backend, run, steps, warmup, kernels)
    flops = 4 * d * hq * t * (t + 1) // 2      # causal-useful multiply-adds * 2, QK^T and PV
    return dict(name=name,
                workload="causal GQA prefill: batch 1, seq 2048, %d/%d heads, d=%d, bf16" % (hq, hkv, d),
                bound="mfma", flops=flops, algorithmic_bytes=(2 * t * hq * d + 2 * t * hkv * d) * 2,
                launches=int(facts.kernel_launches), kernels=kernels, **timed)


def workload_exact2(backend, rng, steps, warmup, hq=40, hkv=8, d=128, name="exact2"):
    """Configuration 2 under the EXACT_F32 contract (F32 tensors, F32 products): the request
    the reference's engine makes.  Not one of the metric's configurations: run by name."""
    t = 2048
    q = backend.tensor("q", B.DTYPE_F32, (t, hq, d), rng.standard_normal((t, hq, d), dtype=np.float32))
    k = backend.tensor("k", B.DTYPE_F32, (t, hkv, d), rng.standard_normal((t, hkv, d), dtype=np.float32))
    v = backend.tensor("v", B.DTYPE_F32, (t, hkv, d), rng.standard_normal((t, hkv, d), dtype=np.float32))
    out = backend.tensor("out", B.DTYPE_F32, (t, hq, d))
    req = backend.attention_requirement(t, t, hq, hkv, d, causal=True)
    run = lambda: backend.attention_execute(req, q, k, v, out)  # noqa: E731
    facts = run()
    kernels = ["yvex_rocm_gqa_f32_tile_%d" % d]
    timed = time_steps(backend, run, steps, warmup, kernels)
    return dict(name=name,
                workload="causal GQA prefill, EXACT_F32 contract: batch 1, seq 2048, %d/%d heads, "
                         "d=%d, f32 in and out" % (hq, hkv, d),
                bound="mfma", flops=4 * d * hq * t * (t + 1) // 2, peak_tflops=MFMA_F32_PEAK_TFLOPS,
                algorithmic_bytes=(2 * t * hq * d + 2 * t * hkv * d) * 4, dtype="f32",
                launches=int(facts.kernel_launches), kernels=kernels, **timed)


def workload_exact1(backend, rng, steps, warmup, hq=32, hkv=8, d=128, name="exact1"):
    """Configuration 1 under the EXACT_F32 contract: the decode step the reference's session
    layer makes (one query token over the cached F32 history).  Run by name."""
    ctx = 4096
    q = backend.tensor("q", B.DTYPE_F32, (1, hq, d), rng.standard_normal((1, hq, d), dtype=np.float32))
    k = backend.tensor("k", B.DTYPE_F32, (ctx, hkv, d), rng.standard_normal((ctx, hkv, d), dtype=np.float32))
    v = backend.tensor("v", B.DTYPE_F32, (ctx, hkv, d), rng.standard_normal((ctx, hkv, d), dtype=np.float32))
    out = backend.tensor("out", B.DTYPE_F32, (1, hq, d))
    req = backend.attention_requirement(1, ctx, hq, hkv, d, causal=True, query_start=ctx - 1)
    work = backend.tensor("workspace", B.DTYPE_I8, (backend.attention_workspace_required(req),))
    backend.workspace_attach(work)
    run = lambda: backend.attention_execute(req, q, k, v, out)  # noqa: E731
    facts = run()
    kernels = ["yvex_rocm_gqa_f32_split" + ("_wide" if d > 128 else "")]
    timed = time_steps(backend, run, steps, warmup, kernels)
    backend.workspace_detach()
    return dict(name=name,
                workload="GQA decode, EXACT_F32 contract: batch 1, %d/%d heads, d=%d, context 4096, "
                         "contiguous f32 KV" % (hq, hkv, d),
                bound="hbm", algorithmic_bytes=2 * ctx * hkv * d * 4 + 2 * hq * d * 4, tokens=ctx,
                dtype="f64", launches=int(facts.kernel_launches), kernels=kernels, **timed)


def workload_decoder_block(backend, rng, steps, warmup):
    """One decode step of the reference's decoder attention block, call for call through the
    reference's own operator slots (src/runtime/decoder.c:1225-1270,
    src/runtime/stateful_attention.c:183-222): split the query/gate projection, rotate and round
    Q and K, two asynchronous copies into the [K | V] history, the write of the token position
    and the two reads of the new rows the session layer makes, attention under EXACT_F32 over
    the strided views, round, sigmoid gate.  Thirteen calls per step on F32 activations; what an
    unchanged caller pays on this backend.  Run by name."""
    hq, hkv, d, ctx, rotary = 32, 8, 128, 4096, 64
    width = hkv * d
    f32 = lambda name, shape, scale=1.0: backend.tensor(  # noqa: E731
        name, B.DTYPE_F32, shape, (rng.standard_normal(shape, dtype=np.float32) * scale))
    qg, k_new, v_new = f32("qg", (1, hq, 2, d)), f32("k-new", (1, hkv, d)), f32("v-new", (1, hkv, d))
    angles = rng.uniform(-3.0, 3.0, (1, rotary))
    cosine = backend.tensor("cos", B.DTYPE_F32, (1, rotary), np.cos(angles).astype(np.float32))
    sine = backend.tensor("sin", B.DTYPE_F32, (1, rotary), np.sin(angles).astype(np.float32))
    history = f32("history", (ctx, 2 * width))
    q, gate = backend.tensor("q", B.DTYPE_F32, (1, hq * d)), backend.tensor("gate", B.DTYPE_F32, (1, hq * d))
    mixer, gated = backend.tensor("mixer", B.DTYPE_F32, (1, hq * d)), backend.tensor("gated", B.DTYPE_F32, (1, hq * d))
    row = (ctx - 1) * 2 * width * 4
    k_slot = history.view(row, B.DTYPE_F32, (width,))
    v_slot = history.view(row + width * 4, B.DTYPE_F32, (width,))
    k_row, v_row = k_new.view(0, B.DTYPE_F32, (width,)), v_new.view(0, B.DTYPE_F32, (width,))
    span = (ctx - 1) * 2 * width + width
    k_view, v_view = history.view(0, B.DTYPE_F32, (span,)), history.view(width * 4, B.DTYPE_F32, (span,))
    req = backend.attention_requirement(1, ctx, hq, hkv, d, causal=True, query_start=ctx - 1,
                                        k_stride=2 * width, v_stride=2 * width)
    work = backend.tensor("workspace", B.DTYPE_I8, (backend.attention_workspace_required(req),))
    backend.workspace_attach(work)

    positions = backend.tensor("positions", B.DTYPE_I64, (ctx,))
    positions.zero()
    position_slot = positions.view((ctx - 1) * 8, B.DTYPE_I64, (1,))
    here = np.array([ctx - 1], dtype=np.int64)

    def run():
        backend.split_interleaved_two_f32(qg, q, gate, 1, hq, d)
        backend.rotary_half_f32(q, cosine, sine, 1, hq, d, rotary)
        backend.bf16_round(q, hq * d)
        backend.rotary_half_f32(k_new, cosine, sine, 1, hkv, d, rotary)
        backend.bf16_round(k_new, width)
        k_slot.copy_from_async(k_row)
        v_slot.copy_from_async(v_row)
        position_slot.write(here)              # stateful_attention.c:222-243: the token positions
        k_new.read()                           # :245-272: the new rows back to the host's delta
        v_new.read()
        facts = backend.attention_execute(req, q, k_view, v_view, mixer)
        backend.bf16_round(mixer, hq * d)
        backend.sigmoid_product_bf16(mixer, gate, gated, hq * d)
        return facts
    run()
    kernels = ["yvex_rocm_gqa_f32_split", "yvex_rocm_rotary_half_plain_f32", "yvex_rocm_bf16_round_f32",
               "yvex_rocm_sigmoid_product_bf16_f32", "yvex_rocm_split_interleaved_two_f32"]
    timed = time_steps(backend, run, steps, warmup, kernels)
    backend.workspace_detach()
    return dict(name="decoder_block",
                workload="one decode step of the reference's decoder attention block, call for call "
                         "(split, rotary and rounding of Q and K, two copies into the [K|V] history, one "
                         "small write and two small reads of the session layer, EXACT_F32 attention "
                         "over 4096 cached tokens, rounding, sigmoid gate): 32/8 heads, d=128, f32 "
                         "activations",
                bound="hbm", algorithmic_bytes=2 * ctx * hkv * d * 4 + 2 * hq * d * 4, tokens=ctx,
                dtype="f64", launches=13, kernels=kernels, **timed)


def workload_decoder_block_fused(backend, rng, steps, warmup):
    """The decode step of workload decoder_block for a caller that keeps bf16 activations and
    uses the two fused entry points: one launch rotates Q where it lies and writes the rotated
    key row and the value row into the [K | V] history, one launch is attention over the
    strided views with the sigmoid gate in its epilogue.  Two launches per step.  Run by name."""
    hq, hkv, d, ctx, rotary = 32, 8, 128, 4096, 64
    width = hkv * d
    bf16 = lambda name, shape: backend.tensor(  # noqa: E731
        name, B.DTYPE_BF16, shape, random_bf16(rng, int(np.prod(shape))))
    q, gate = bf16("q", (1, hq, d)), bf16("gate", (1, hq, d))
    k_new, v_new = bf16("k-new", (1, hkv, d)), bf16("v-new", (1, hkv, d))
    angles = rng.uniform(-3.0, 3.0, (1, rotary))
    cosine = backend.tensor("cos", B.DTYPE_F32, (1, rotary), np.cos(angles).astype(np.float32))
    sine = backend.tensor("sin", B.DTYPE_F32, (1, rotary), np.sin(angles).astype(np.float32))
    history = bf16("history", (ctx, 2 * width))
    gated = backend.tensor("gated", B.DTYPE_BF16, (1, hq, d))
    span = (ctx - 1) * 2 * width + width
    k_view, v_view = history.view(0, B.DTYPE_BF16, (span,)), history.view(width * 2, B.DTYPE_BF16, (span,))
    req = backend.attention_requirement(1, ctx, hq, hkv, d, causal=True, query_start=ctx - 1,
                                        dtype=B.DTYPE_BF16, contract=B.NUMERIC_BF16_F32_ACCUMULATE,
                                        k_stride=2 * width, v_stride=2 * width)
    work = backend.tensor("workspace", B.DTYPE_I8, (backend.attention_workspace_required(req),))
    backend.workspace_attach(work)

    def run():
        backend.history_append_execute(k_new, v_new, k_view, v_view, ctx - 1, hkv, head_dimension=d,
                                       cosine=cosine, sine=sine, rotary_dimension=rotary,
                                       key_token_stride=2 * width, value_token_stride=2 * width,
                                       query=q, query_heads=hq)
        return backend.attention_execute(req, q, k_view, v_view, gated, gate=gate)
    facts = run()
    kernels = ["yvex_rocm_decode_rows_bf16_team", "yvex_rocm_history_append_bf16"]
    timed = time_steps(backend, run, steps, warmup, kernels)
    backend.workspace_detach()
    return dict(name="decoder_block_fused",
                workload="one decode step of the decoder attention block through the fused entry "
                         "points (rotary of Q and K and both history rows in one launch, attention "
                         "over 4096 cached tokens with the sigmoid gate in its epilogue): 32/8 heads, "
                         "d=128, bf16 activations",
                bound="hbm", algorithmic_bytes=2 * ctx * hkv * d * 2 + 3 * hq * d * 2, tokens=ctx,
                launches=1 + int(facts.kernel_launches), kernels=kernels, **timed)


def workload_mla5(backend, rng, steps, warmup):
    batch, heads, kd, vd, page, ctx = 16, 128, 576, 512, 64, 8192
    pages_each = ctx // page
    pool_pages = batch * pages_each
    table = rng.permutation(pool_pages).astype(np.int32).reshape(batch, pages_each)
    contexts = np.full(batch, ctx, dtype=np.int32)
    pool = backend.tensor("latent-pages", B.DTYPE_BF16, (pool_pages, page, kd),
                          random_bf16(rng, pool_pages * page * kd))
    q = backend.tensor("q", B.DTYPE_BF16, (batch, heads, kd), random_bf16(rng, batch * heads * kd))
    tt = backend.tensor("table", B.DTYPE_I32, table.shape, table)
    tc = backend.tensor("ctx", B.DTYPE_I32, contexts.shape, contexts)
    out = backend.tensor("out", B.DTYPE_BF16, (batch, heads, vd))
    lse = backend.tensor("lse", B.DTYPE_F32, (batch, heads))
    req = backend.mla_requirement(batch, heads, kd, vd, page, pool_pages, pages_each, ctx)
    work = backend.tensor("workspace", B.DTYPE_I8, (backend.mla_decode_workspace_required(req),))
    backend.workspace_attach(work)
    run = lambda: backend.mla_decode_execute(req, q, pool, tt, tc, out, lse)  # noqa: E731
    facts = run()
    kernels = ["yvex_rocm_mla_decode_bf16", "yvex_rocm_decode_merge"]
    timed = time_steps(backend, run, steps, warmup, kernels)
    backend.workspace_detach()
    algo = batch * ctx * kd * 2 + batch * heads * (kd + vd) * 2 + table.size * 4 + batch * heads * 4
    assert np.all(np.isfinite(lse.read()))
    return dict(name="mla5",
                workload="absorbed MLA decode: batch 16, 128 heads, latent 512 + rope 64, "
                         "context 8192 in 64-token pages",
                bound="hbm", algorithmic_bytes=algo, flops=batch * heads * ctx * 2 * (kd + vd),
                launches=int(facts.kernel_launches), kernels=kernels, **timed)


def workload_append(backend, rng, steps, warmup, q8=False):
    """The KV page writer on a prefill-sized batch: 16 sessions x 2048 new tokens, 8 kv heads,
    d=128, rotate-half on the whole key row, unaligned start positions.  Not one of the
    metric's configurations: run by name."""
    sessions, hkv, d, page, new = 16, 8, 128, 16, 2048
    starts = rng.integers(0, 4096, size=sessions).astype(np.int32)
    counts = np.full(sessions, new, np.int32)
    stride = int((starts.max() + new + page - 1) // page)
    pool_pages = sessions * stride
    table = rng.permutation(pool_pages).astype(np.int32).reshape(sessions, stride)
    total = sessions * new
    block = 2176 if q8 else 4096
    pool_bytes = pool_pages * hkv * block
    pool_dtype = B.DTYPE_I8 if q8 else B.DTYPE_BF16
    elems = pool_bytes // B.DTYPE_BYTES[pool_dtype]
    angles = rng.uniform(-3.0, 3.0, size=(total, d)).astype(np.float32)
    t = [backend.tensor("k-new", B.DTYPE_BF16, (total, hkv, d), random_bf16(rng, total * hkv * d)),
         backend.tensor("v-new", B.DTYPE_BF16, (total, hkv, d), random_bf16(rng, total * hkv * d)),
         backend.tensor("rows", B.DTYPE_I32, (sessions,), (np.arange(sessions) * new).astype(np.int32)),
         backend.tensor("starts", B.DTYPE_I32, (sessions,), starts),
         backend.tensor("counts", B.DTYPE_I32, (sessions,), counts),
         backend.tensor("table", B.DTYPE_I32, table.shape, table),
         backend.tensor("k-pages", pool_dtype, (elems,)),
         backend.tensor("v-pages", pool_dtype, (elems,))]
    t[6].zero()
    t[7].zero()
    cosine = backend.tensor("cos", B.DTYPE_F32, angles.shape, np.cos(angles))
    sine = backend.tensor("sin", B.DTYPE_F32, angles.shape, np.sin(angles))
    storage = B.KV_Q8_0 if q8 else B.KV_BF16
    run = lambda: backend.kv_append_execute(*t, hkv, pool_pages, new, storage=storage,  # noqa: E731
                                            cosine=cosine, sine=sine, rotary_dimension=d)
    facts = run()
    kernel = "yvex_rocm_kv_append_q8_0" if q8 else "yvex_rocm_kv_append_bf16"
    kernels = [kernel]
    timed = time_steps(backend, run, steps, warmup, kernels)
    # per token: K and V rows in (bf16), both page rows out, half a cos and half a sin row
    algo = total * (2 * hkv * d * 2 + 2 * hkv * (136 if q8 else 256) + d * 4) + 3 * sessions * 4
    return dict(name="append_q8_0" if q8 else "append_bf16",
                workload="KV page writer, %s pages: 16 sessions x 2048 new tokens, 8 kv heads, "
                         "d=128, rotary 128, unaligned starts" % ("Q8_0" if q8 else "bf16"),
                bound="hbm", algorithmic_bytes=algo, tokens=total,
                launches=int(facts.kernel_launches), kernels=kernels, **timed)


def workload_history_append(backend, rng, steps, warmup):
    """The token-major history writer on a prompt: 8192 new tokens, 8 kv heads, d=128,
    rotate-half on the whole key row, into an interleaved [K | V] history that lives in a
    reserved address range committed for these rows.  Not one of the metric's
    configurations: run by name."""
    hkv, d, new, first = 8, 128, 8192, 1000
    width = hkv * d
    used = first + new
    history = backend.reserve("history", B.DTYPE_BF16, (32768, 2 * width))
    history.commit(0, used * 2 * width * 2)
    count = (used - 1) * 2 * width + width
    kh = history.view(0, B.DTYPE_BF16, (count,))
    vh = history.view(2 * width, B.DTYPE_BF16, (count,))
    angles = rng.uniform(-3.0, 3.0, size=(new, d)).astype(np.float32)
    key = backend.tensor("k-new", B.DTYPE_BF16, (new, hkv, d), random_bf16(rng, new * hkv * d))
    value = backend.tensor("v-new", B.DTYPE_BF16, (new, hkv, d), random_bf16(rng, new * hkv * d))
    cosine = backend.tensor("cos", B.DTYPE_F32, angles.shape, np.cos(angles))
    sine = backend.tensor("sin", B.DTYPE_F32, angles.shape, np.sin(angles))
    run = lambda: backend.history_append_execute(  # noqa: E731
        key, value, kh, vh, first, hkv, cosine=cosine, sine=sine, rotary_dimension=d,
        key_token_stride=2 * width, value_token_stride=2 * width)
    facts = run()
    kernels = ["yvex_rocm_history_append_bf16"]
    timed = time_steps(backend, run, steps, warmup, kernels)
    # per token: K and V rows in, both out, half a cos and half a sin row
    algo = new * (4 * width * 2 + d * 4)
    return dict(name="history_append",
                workload="token-major history writer: 8192 new tokens behind 1000, 8 kv heads, "
                         "d=128, rotary 128, interleaved [K|V] rows in a reserved address range",
                bound="hbm", algorithmic_bytes=algo, tokens=new,
                launches=int(facts.kernel_launches), kernels=kernels, **timed)


def copy_reference(backend, steps):
    """A device-to-device copy of known size: the scale for the FETCH_SIZE / WRITE_SIZE
    counters.  Not a workload of the metric; run as --workload copy."""
    nbytes = 1 << 30
    src = backend.tensor("copy-src", B.DTYPE_I8, (nbytes,))
    dst = backend.tensor("copy-dst", B.DTYPE_I8, (nbytes,))
    src.zero()
    backend.sync()
    backend.timing_begin()
    for _ in range(steps):
        dst.copy_from(src)
    ms = backend.timing_end() / steps
    return dict(bytes_read=nbytes, bytes_written=nbytes, ms_per_copy=ms,
                gbs=2 * nbytes / (ms * 1e-3) / 1e9)


WORKLOADS = {
    "prefill2": workload_prefill2,
    "decode1": workload_decode1,
    "paged3": lambda b, r, s, w: workload_paged(b, r, s, w, q8=False),
    "paged4": lambda b, r, s, w: workload_paged(b, r, s, w, q8=True),
    "mla5": workload_mla5,
}
# measured by name only (rows next to the metric's path, not configurations of the metric)
EXTRA_WORKLOADS = {
    "append_bf16": lambda b, r, s, w: workload_append(b, r, s, w, q8=False),
    "append_q8_0": lambda b, r, s, w: workload_append(b, r, s, w, q8=True),
    "history_append": workload_history_append,
    "paged3_p64": lambda b, r, s, w: workload_paged(b, r, s, w, q8=False, page=64),
    "paged4_p64": lambda b, r, s, w: workload_paged(b, r, s, w, q8=True, page=64),
    "exact2": workload_exact2,
    "exact1": workload_exact1,
    # the reference's own Qwen attention geometry (24/4 heads, head dimension 256) and a narrow one
    "prefill_d256": lambda b, r, s, w: workload_prefill2(b, r, s, w, hq=24, hkv=4, d=256, name="prefill_d256"),
    "prefill_d64": lambda b, r, s, w: workload_prefill2(b, r, s, w, hq=16, hkv=4, d=64, name="prefill_d64"),
    "exact2_d256": lambda b, r, s, w: workload_exact2(b, r, s, w, hq=24, hkv=4, d=256, name="exact2_d256"),
    "exact1_d256": lambda b, r, s, w: workload_exact1(b, r, s, w, hq=24, hkv=4, d=256, name="exact1_d256"),
    "decode_d256": lambda b, r, s, w: workload_decode1(b, r, s, w, hq=24, hkv=4, d=256, name="decode_d256"),
    "decode_d64": lambda b, r, s, w: workload_decode1(b, r, s, w, hq=16, hkv=4, d=64, name="decode_d64"),
    "paged_d256": lambda b, r, s, w: workload_paged(b, r, s, w, hq=24, hkv=4, d=256, name="paged_d256"),
    "paged_d64": lambda b, r, s, w: workload_paged(b, r, s, w, hq=16, hkv=4, d=64, name="paged_d64"),
    "decoder_block": workload_decoder_block,
    "decoder_block_fused": workload_decoder_block_fused,
}
SEEDS = {"decode1": 1, "prefill2": 2, "paged3": 3, "paged4": 4, "mla5": 5, "append_bf16": 6,
         "append_q8_0": 7, "exact2": 8, "exact1": 9, "history_append": 10, "paged3_p64": 3, "paged4_p64": 4,
         "prefill_d256": 11, "prefill_d64": 12, "paged_d256": 13, "paged_d64": 14, "decoder_block": 15,
         "decoder_block_fused": 15, "decode_d256": 16, "decode_d64": 17,
         "exact2_d256": 18, "exact1_d256": 19}


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def measured_traffic(name, kernel):
    """HBM bytes per launch of `kernel` in workload `name`, from the committed counter summary
    (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs, each scaled by what the same counter
    reads for a device copy of known size).  Not measured in this process: None when the file
    has no entry for this kernel."""
    try:
        with open(TRAFFIC_FILE, encoding="utf-8") as stream:
            table = json.load(stream)
    except (OSError, ValueError):
        return None
    entry = table.get("workloads", {}).get(name, {}).get(kernel)
    return None if entry is None else int(entry["hbm_bytes"])


def roofline(result):
    """Roofline record of the dominant kernel.  `achieved` is the algorithmic bytes (or flops)
    of one launch over that kernel's own mean duration and `frac` (= `kernel_frac`) its share
    of the published peak.  `step_achieved` / `step_frac` are the same quantity over the whole
    step, every launch and the gaps between them included: that is what `value` reports.  Both
    are as measured; the event pair around a single launch costs a few microseconds, so for a
    step of one short kernel the per-launch figure can come out longer than the step."""
    kernel = result["kernels"][0]
    if kernel not in result["kernel_ms"]:
        sys.exit("bench.py: kernel %s was not launched by workload %s" % (kernel, result["name"]))
    seconds = result["kernel_ms"][kernel] * 1e-3
    step_seconds = result["ms"] * 1e-3
    if result["bound"] == "hbm":
        work, scale, peak, unit = result["algorithmic_bytes"], 1e9, HBM_PEAK_GBS, "GB/s"
    else:
        work, scale, unit = result["flops"], 1e12, "TFLOP/s"
        peak = result.get("peak_tflops", MFMA_BF16_PEAK_TFLOPS)
    achieved, step_achieved = work / seconds / scale, work / step_seconds / scale
    return dict(bound=result["bound"], achieved=achieved, peak=peak, unit=unit, frac=achieved / peak,
                traffic=measured_traffic(result["name"], kernel),
                traffic_source="profiles/hbm_traffic.json (rocprofv3 --pmc, not this run)",
                kernel=kernel, kernel_us=seconds * 1e6, kernel_frac=achieved / peak,
                step_us=step_seconds * 1e6, step_achieved=step_achieved,
                step_frac=step_achieved / peak,
                kernels_us={k: v * 1e3 for k, v in result["kernel_ms"].items()})


def repeat_for(seconds, call, least=3):
    """Calls `call` at least `least` times and until `seconds` of wall time have passed;
    returns (runs, median seconds of one run, total seconds)."""
    durations, t0 = [], time.perf_counter()
    while True:
        c0 = time.perf_counter()
        rc = call()
        durations.append(time.perf_counter() - c0)
        assert rc == 0
        if len(durations) >= least and time.perf_counter() - t0 >= seconds:
            return len(durations), float(np.median(durations)), time.perf_counter() - t0


def reference_operator_leg(rng, keys, heads, d, budget=2.0):
    """The reference's own CPU operator (yvex_backend_op_attention, compiled from the reference's
    sources into oracle/_ref, single thread, one query head per call over F32 rows): seconds
    per head over `keys` keys, median of the runs that fit `budget`.  None where oracle/_ref was
    not built."""
    import ctypes
    from oracle_binding import load_reference
    ref = load_reference()
    if ref is None:
        return None
    f32p = ctypes.POINTER(ctypes.c_float)
    q = rng.standard_normal(d, dtype=np.float32)
    k = rng.standard_normal((keys, d), dtype=np.float32)
    v = rng.standard_normal((keys, d), dtype=np.float32)
    out = np.zeros(d, np.float32)
    score, prob = np.zeros(keys, np.float32), np.zeros(keys, np.float32)
    ptr = lambda a: a.ctypes.data_as(f32p)  # noqa: E731

    def one_head():
        rc = ref.yvref_op_attention(ptr(q), ptr(k), ptr(v), keys, keys - 1, d,
                                    np.float32(1.0 / np.sqrt(d)), 1, ptr(score), ptr(prob), ptr(out))
        assert rc == 0
        return rc
    runs, dt, spent = repeat_for(budget, one_head)
    return dict(seconds_per_head=dt, keys=keys, head_dim=d, cores=1, kind="reference",
                sample="yvex_backend_op_attention of the compiled reference, one query head over %d "
                       "F32 keys, single thread, median of %d runs (%.1f s)" % (keys, runs, spent),
                heads_of_the_workload=heads)


def cpu_baseline(name, budget=6.0):
    """The oracle (a port of the reference CPU operator, all host threads) timed on a bounded
    sample of the same workload: the sample is repeated at least three times and for about `budget` seconds, and the median run
    is reported."""
    from oracle_binding import Oracle
    oracle = Oracle()
    rng = np.random.default_rng(SEEDS[name])
    threads = oracle.threads
    if name in ("paged3", "paged4"):
        sessions, hq, hkv, d, page = 4, 32, 8, 128, 16
        contexts = np.full(sessions, 8192, dtype=np.int32)
        pool_pages = int(contexts.sum()) // page
        table = rng.permutation(pool_pages).astype(np.int32).reshape(sessions, -1)
        k = bf16_bits(rng.standard_normal((pool_pages, page, hkv, d), dtype=np.float32))
        v = bf16_bits(rng.standard_normal((pool_pages, page, hkv, d), dtype=np.float32))
        q = bf16_bits(rng.standard_normal((sessions, hq, d), dtype=np.float32))
        q8 = name == "paged4"
        if q8:
            k = oracle.q8_0_encode_rows(oracle.bf16_decode(k))
            v = oracle.q8_0_encode_rows(oracle.bf16_decode(v))
        runs, dt, spent = repeat_for(budget, lambda: oracle.paged_decode(q, k, v, table, contexts, hkv,
                                                                  page, q8=q8)[0])
        per_token = 2 * hkv * (136 if q8 else 256)
        leg = reference_operator_leg(rng, 8192, hq, d)
        if leg:   # the same bytes per token if one thread ran every query head of a session
            leg.update(value=8192 * per_token / (leg["seconds_per_head"] * hq) / 1e9, unit="GB/s")
        return dict(value=int(contexts.sum()) * per_token / dt / 1e9, unit="GB/s", cores=threads,
                    kind="port", sample="4 sessions x 8192 tokens of the same shape, median of "
                                        "%d runs (%.1f s)" % (runs, spent), reference_operator=leg)
    if name == "decode1":
        q = bf16_bits(rng.standard_normal((1, 32, 128), dtype=np.float32))
        k = bf16_bits(rng.standard_normal((4096, 8, 128), dtype=np.float32))
        v = bf16_bits(rng.standard_normal((4096, 8, 128), dtype=np.float32))
        runs, dt, spent = repeat_for(budget / 2, lambda: oracle.gqa_bf16(q, k, v, query_start=4095)[0])
        leg = reference_operator_leg(rng, 4096, 32, 128)
        if leg:
            leg.update(value=(2 * 4096 * 8 * 128 * 2) / (leg["seconds_per_head"] * 32) / 1e9, unit="GB/s")
        return dict(value=(2 * 4096 * 8 * 128 * 2) / dt / 1e9, unit="GB/s", cores=threads,
                    kind="port", sample="the full workload, median of %d runs (%.1f s)" %
                                        (runs, spent), reference_operator=leg)
    if name == "prefill2":
        t, hq, hkv, d = 1024, 40, 8, 128
        q = bf16_bits(rng.standard_normal((t, hq, d), dtype=np.float32))
        k = bf16_bits(rng.standard_normal((t, hkv, d), dtype=np.float32))
        v = bf16_bits(rng.standard_normal((t, hkv, d), dtype=np.float32))
        runs, dt, spent = repeat_for(budget, lambda: oracle.gqa_bf16(q, k, v, query_start=0)[0])
        return dict(value=4 * d * hq * t * (t + 1) // 2 / dt / 1e12, unit="TFLOP/s", cores=threads,
                    kind="port", sample="the first 1024 tokens of the same shape, median of %d runs "
                                        "(%.1f s)" % (runs, spent))
    if name == "exact2":
        t, hq, hkv, d = 512, 40, 8, 128
        q = rng.standard_normal((t, hq, d), dtype=np.float32)
        k = rng.standard_normal((t, hkv, d), dtype=np.float32)
        v = rng.standard_normal((t, hkv, d), dtype=np.float32)
        runs, dt, spent = repeat_for(budget, lambda: oracle.gqa(q, k, v)[0])
        return dict(value=4 * d * hq * t * (t + 1) // 2 / dt / 1e12, unit="TFLOP/s", cores=threads,
                    kind="port", sample="the first 512 tokens of the same shape, median of %d runs "
                                        "(%.1f s)" % (runs, spent))
    if name == "exact1":
        q = rng.standard_normal((1, 32, 128), dtype=np.float32)
        k = rng.standard_normal((4096, 8, 128), dtype=np.float32)
        v = rng.standard_normal((4096, 8, 128), dtype=np.float32)
        runs, dt, spent = repeat_for(budget / 2, lambda: oracle.gqa(q, k, v, query_start=4095)[0])
        return dict(value=(2 * 4096 * 8 * 128 * 4) / dt / 1e9, unit="GB/s", cores=threads, kind="port",
                    sample="the full workload, median of %d runs (%.1f s)" % (runs, spent))
    if name == "mla5":
        batch, heads, kd, vd, page, ctx = 2, 128, 576, 512, 64, 4096
        pages = batch * ctx // page
        table = rng.permutation(pages).astype(np.int32).reshape(batch, -1)
        pool = bf16_bits(rng.standard_normal((pages, page, kd), dtype=np.float32))
        q = bf16_bits(rng.standard_normal((batch, heads, kd), dtype=np.float32))
        contexts = np.full(batch, ctx, np.int32)
        runs, dt, spent = repeat_for(budget, lambda: oracle.mla_decode(q, pool, table, contexts, vd,
                                                                page)[0])
        return dict(value=batch * ctx * kd * 2 / dt / 1e9, unit="GB/s", cores=threads, kind="port",
                    sample="2 batch elements x 4096 tokens of the same shape, median of %d runs "
                           "(%.1f s)" % (runs, spent))
    return None


METRIC = "decode attn HBM GB/s (% of peak); prefill attn TFLOPS (% MFMA peak), 1 GPU"


def main():
    global SPIN_UP_SECONDS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all",
                    help="one workload name, or 'all' (default): every configuration, with "
                         "the paged bf16 decode as the headline value")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--spin-up", type=float, default=SPIN_UP_SECONDS,
                    help="seconds of untimed steps before the warm-up steps of each workload "
                         "(the part raises its clocks only under sustained load); printed as "
                         "spin_up_s")
    args = ap.parse_args()
    SPIN_UP_SECONDS = args.spin_up
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported "
                 "(attention shards by session or head without exchange)" % args.gpus)
    if args.workload == "copy":
        backend = Backend()
        print(json.dumps({"copy_reference": copy_reference(backend, min(args.steps, 10))}))
        backend.close()
        return
    names = list(WORKLOADS) if args.workload == "all" else [args.workload]
    headline = "paged3" if args.workload == "all" else args.workload
    results = {}
    for name in names:
        backend = Backend()
        if backend.status != B.STATUS_READY:
            sys.exit("bench.py: ROCm backend is not ready: %s" % backend.report().rejection.decode())
        rng = np.random.default_rng(SEEDS[name])
        results[name] = {**WORKLOADS, **EXTRA_WORKLOADS}[name](backend, rng, args.steps, args.warmup)
        backend.close()
    # what the part sustains on a plain streaming read and on a copy (the library's own probe):
    # context for the roofline fractions, which are quoted against the published 8 TB/s
    backend = Backend()
    evidence = backend.bandwidth_probe()
    backend.close()
    device_probe = {"hbm_stream_read_gbs": evidence.sustainable_read_bytes_per_second / 1e9,
                    "device_copy_gbs": evidence.sustainable_copy_bytes_per_second / 1e9,
                    "working_set_bytes": int(evidence.working_set_bytes)}
    head = results[headline]
    roof = roofline(head)
    cpu = {} if args.no_cpu else {n: cpu_baseline(n) for n in names}
    line = {
        "metric": METRIC,
        "value": roof["step_achieved"],
        "unit": roof["unit"],
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "spin_up_s": SPIN_UP_SECONDS,
        "ms_per_step": head["ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": head.get("dtype", "bf16"), "data": "synthetic",
        "config": {"workload": head["workload"], "name": head["name"],
                   "kernel_launches_per_step": head["launches"]},
        "roofline": roof,
        "benchmark_record": head["record"],
        "cpu_baseline": cpu.get(headline),
        "device_probe": device_probe,
        # the metric has two halves; `value` carries the first (decode, HBM GB/s), this the
        # second (causal prefill, TFLOP/s), when that workload ran
        "prefill": ({"metric": "prefill attn TFLOPS (% MFMA peak)",
                     "value": roofline(results["prefill2"])["step_achieved"], "unit": "TFLOP/s",
                     "ms_per_step": results["prefill2"]["ms"],
                     "config": {"workload": results["prefill2"]["workload"]},
                     "roofline": roofline(results["prefill2"]),
                     "cpu_baseline": cpu.get("prefill2")} if "prefill2" in results else None),
        "workloads": {n: dict(workload=r["workload"], ms_per_step=r["ms"],
                              wall_ms_per_step=r["wall_ms"],
                              value=roofline(r)["step_achieved"], unit=roofline(r)["unit"],
                              roofline=roofline(r), benchmark_record=r["record"],
                              cpu_baseline=cpu.get(n)) for n, r in results.items()},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
