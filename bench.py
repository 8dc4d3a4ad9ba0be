#!/usr/bin/env python3
"""Benchmark of the NAtS-L hybrid-layer forward (selector + routing + softmax branch + Gated DeltaNet
branch) on one MI355X.  A step is one pass of that path over one synthetic batch resident in HBM.

Prints ONE JSON line: tokens/s of the whole step, the roofline of the dominant kernel (the sparse
softmax kernel, MFMA-bound) from HIP events recorded on the stream it is launched on, and a
host-CPU baseline (the fp32 oracle on a bounded sample of the same workload).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: B, T, H, K, V, attention rate, selector block
    "hybrid_gdn_B8_T8192_H16_d128_p25": dict(B=8, T=8192, H=16, K=128, V=128, p_attn=0.25, block=64),
    "gdn_only_B4_T4096_H16_d128": dict(B=4, T=4096, H=16, K=128, V=128, p_attn=0.0, block=64),
    "hybrid_gdn_B1_T65536_H32_d128_p10": dict(B=1, T=65536, H=32, K=128, V=128, p_attn=0.10, block=64),
    # the Mamba2-SSD variant: K = state dim (B, C shared by all heads), V = head dim, selector block 256
    "hybrid_mamba_B4_T8192_H32_N128_d64_p25": dict(B=4, T=8192, H=32, K=128, V=64, p_attn=0.25, block=256, kind="mamba"),
}
# decode: one new token per sequence on cached states, the attention branch over the cached keys/values of the
# attention-typed blocks (p_attn of the context) plus the current block; not the headline metric
DECODE_WORKLOADS = {
    "decode_gdn_B8_ctx8192_H16_d128_p25": dict(B=8, ctx=8192, H=16, K=128, V=128, p_attn=0.25, block=64, n_in_block=17),
}
# cache hand-off after a prefill: keep the attention-typed blocks of every (sequence, head); not the headline metric
CACHE_WORKLOADS = {
    "kv_compact_B8_T8192_H16_d128_p25": dict(B=8, T=8192, H=16, K=128, V=128, p_attn=0.25, block=64),
}
# backward of the softmax branch at the headline shape (training); not the headline metric
BACKWARD_WORKLOADS = {
    "softmax_bwd_B8_T8192_H16_d128_p25": dict(B=8, T=8192, H=16, K=128, V=128, p_attn=0.25, block=64),
}
# backward of the Gated DeltaNet branch at the headline shape (training); not the headline metric
LINEAR_BACKWARD_WORKLOADS = {
    "gdn_bwd_B8_T8192_H16_d128_p25": dict(B=8, T=8192, H=16, K=128, V=128, p_attn=0.25, block=64),
    "gdn_bwd_B8_T4096_H6_K128_V256_p25": dict(B=8, T=4096, H=6, K=128, V=256, p_attn=0.25, block=64),     # the 340M geometry
    "gdn_bwd_B8_T4096_H6_K192_V384_p25": dict(B=8, T=4096, H=6, K=192, V=384, p_attn=0.25, block=64),     # the 760M geometry
    "mamba_bwd_B4_T8192_H32_N128_d64_p25": dict(B=4, T=8192, H=32, K=128, V=64, p_attn=0.25, block=256, kind="mamba"),
}
# a whole Gated-DeltaNet layer at the published 340M geometry (hidden 1024, 6 heads of 128 / 256, attention view 12 heads of
# 64 / 128): forward, or forward + backward; not the headline metric
LAYER_WORKLOADS = {
    "layer_gdn_340M_B8_T4096_fwd": dict(B=8, T=4096, train=False),
    "layer_gdn_340M_B8_T4096_train": dict(B=8, T=4096, train=True),
}
PEAK_BF16_MFMA_TFLOPS = 2500.0   # MI355X dense bf16
PEAK_HBM_GBS = 8000.0


def selector_bias(p_attn):
    """bias on the linear op's logit so that P(attention) = p_attn for N(0,1) logit pairs: b = -sqrt(2)*Phi^-1(p)."""
    if p_attn <= 0.0:
        return 30.0
    if p_attn >= 1.0:
        return -30.0
    from statistics import NormalDist
    return -math.sqrt(2.0) * NormalDist().inv_cdf(p_attn)


def make_inputs(w, torch, device):
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(0)
    B, T, H, K, V = w["B"], w["T"], w["H"], w["K"], w["V"]
    if w.get("kind") == "mamba":
        # C (as q) and B (as k) ~ N(0,1), one group shared by all heads; X ~ N(0,1); log-decay dt * A with
        # dt = softplus(N(0,1) - 4), A = -exp(U(0, log 16)) per head.  The linear branch takes X * dt as its values, the
        # attention branch the unscaled X (src/nats/layers/natsl_attn_mamba2.py:391-393, :473).
        q = torch.randn(B, T, 1, K, generator=g).expand(B, T, H, K).contiguous().bfloat16()
        k = torch.randn(B, T, 1, K, generator=g).expand(B, T, H, K).contiguous().bfloat16()
        x = torch.randn(B, T, H, V, generator=g)
        beta = torch.ones(B, T, H).bfloat16()
        dt = F.softplus(torch.randn(B, T, H, generator=g) - 4.0)
        gl = -torch.exp(torch.rand(H, generator=g) * math.log(16.0)) * dt
        v, v_l = x.bfloat16(), (x * dt[..., None]).bfloat16()
    else:
        q = torch.randn(B, T, H, K, generator=g).bfloat16()
        k = torch.randn(B, T, H, K, generator=g).bfloat16()
        v = torch.randn(B, T, H, V, generator=g).bfloat16()
        beta = torch.sigmoid(torch.randn(B, T, H, generator=g)).bfloat16()
        gl = -F.softplus(torch.randn(B, T, H, generator=g))
        v_l = v
    logits = torch.randn(B, T // w["block"], H, 2, generator=g)
    logits[..., 1] += selector_bias(w["p_attn"])
    logits = logits.bfloat16()
    host = dict(q=q, k=k, v=v, v_l=v_l, beta=beta, g=gl, logits=logits)
    dev = {n: t.to(device) for n, t in host.items()}
    return host, dev


def csrc_sha():
    """sha256 over the kernel sources the library is built from: names the code a counter measurement belongs to."""
    import hashlib
    d = os.path.join(ROOT, "neuralattentionsearchlinear_amd", "csrc")
    h = hashlib.sha256()
    for f in sorted(os.listdir(d)):
        if f.endswith((".hip", ".h")):
            h.update(f.encode())
            h.update(open(os.path.join(d, f), "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(workload):
    """HBM bytes per launch (read + written) per kernel, from the FETCH_SIZE / WRITE_SIZE counter runs of this script
    whose summary is kept in profiles/bench_<workload>.md on a line `traffic-json: {...}`.  The line names the kernel
    sources it was measured on (csrc_sha); counters of other sources are stale and are not reported."""
    path = os.path.join(ROOT, "profiles", f"bench_{workload}.md")
    if not os.path.exists(path):
        return None, "no counter summary under profiles/"
    for line in open(path):
        if line.startswith("traffic-json:"):
            rec = json.loads(line[len("traffic-json:"):])
            if rec.get("csrc_sha") != csrc_sha():
                return None, f"profiles/{os.path.basename(path)} was measured on other kernel sources ({rec.get('csrc_sha')})"
            return rec, f"profiles/{os.path.basename(path)} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, csrc_sha {rec['csrc_sha']})"
    return None, "no traffic-json line in the counter summary"


def clock_probe(torch, device):
    """Shader clock and matrix rate of a pure v_mfma_f32_32x32x16_bf16 loop, right after the timed steps.  The probe kernel
    is a benchmark aid in a library of its own (csrc/libnatsl_bench.so, built with the package), not part of the C ABI."""
    import ctypes
    from neuralattentionsearchlinear_amd import _build, _capi
    if not os.path.exists(_build.BENCH_LIB):
        return dict(note="csrc/libnatsl_bench.so is not built: no clock measurement")
    L = ctypes.CDLL(_build.BENCH_LIB)
    L.natsl_bench_mfma_clock_probe.restype = ctypes.c_int
    L.natsl_bench_mfma_clock_probe.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    n_wg, iters = 2 * cus, 40000
    out = torch.zeros(2 * n_wg, dtype=torch.int64, device=device)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    assert L.natsl_bench_mfma_clock_probe(_capi.ptr(out), n_wg, 2000, _capi.stream_ptr(device)) == 0
    ev[0].record()
    assert L.natsl_bench_mfma_clock_probe(_capi.ptr(out), n_wg, iters, _capi.stream_ptr(device)) == 0
    ev[1].record()
    torch.cuda.synchronize()
    ms = ev[0].elapsed_time(ev[1])
    o = out.cpu().view(n_wg, 2).double()
    mhz = float((o[:, 0] / o[:, 1]).median()) * 100.0
    tflops = n_wg * 4 * iters * 4 * 32768.0 / (ms * 1e-3) / 1e12
    return dict(clock_mhz_under_load=mhz, mfma_loop_tflops=tflops,
                note="pure 32x32x16 bf16 MFMA loop, 2 workgroups x 4 waves per CU, launched right after the timed steps")


def softmax_kernel_name(B, T, H, block):
    """The kernel natsl_softmax_sparse_fwd runs for this problem, as the library itself reports it."""
    from neuralattentionsearchlinear_amd import _capi
    v = _capi.lib().natsl_softmax_fwd_variant(B, T, H, H, block, 0)
    return {0: "softmax_sparse_fwd_kernel<4 waves>", 1: "softmax_sparse_fwd_kernel<8 waves>", 2: "softmax_stream_kernel"}.get(v, f"unknown ({v})")


def softmax_flops(types, T, block, K, V):
    """2(K+V) * sum over queries of visible keys, mode 'all': own block causally + earlier attention blocks."""
    a = types[..., 0].float().round()                     # [B,NB,HN]
    prior = a.cumsum(1) - a
    n = float(block)
    return 2.0 * (K + V) * float((n * (n + 1) / 2 + n * block * prior).sum())


def gdn_flops(types, K, V, C=64, per_block=1):
    """per 64-token chunk and head: the two Gram products, the solve, w S, T X, q S, P v_new and the state update (kept for
    chunks of blocks typed linear).  types are per selector block of per_block chunks."""
    lin = types[..., 1].float().round()
    n_all, n_lin = float(lin.numel()) * per_block, float(lin.sum()) * per_block
    per = 2 * C * C * (3 * K + 2 * V) + 6 * C * K * V + (2.0 / 3.0) * C ** 3
    return per * n_all - 2 * C * K * V * (n_all - n_lin)


def mamba_flops(types, K, V, C=64, per_block=1):
    """per chunk and head: q k^T, P v, q S, and the state update for chunks of blocks typed linear."""
    lin = types[..., 1].float().round()
    n_all, n_lin = float(lin.numel()) * per_block, float(lin.sum()) * per_block
    return (2 * C * C * (K + V) + 2 * C * K * V) * n_all + 2 * C * K * V * n_lin


def cpu_baseline(host, w, types_host, torch, max_heads=None, max_batch=None):
    """fp32 oracle on a batch/head slice of the workload (full sequence length), on the host cores."""
    from oracle import mixed
    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    torch.set_num_threads(threads)
    H = w["H"] if max_heads is None else min(w["H"], max_heads)
    Bs = w["B"] if max_batch is None else min(w["B"], max_batch)
    sl = lambda t: t[:Bs, :, :H].contiguous()
    q, k, v, v_l, beta, g = (sl(host[n]) for n in ("q", "k", "v", "v_l", "beta", "g"))
    ty = types_host[:Bs, :, :H].contiguous()
    t0 = time.perf_counter()
    if w.get("kind") == "mamba":
        mixed.mixed_attn_mamba(q, k, v, q, k, v_l, None, g, ty, scale_lattn=1.0, ops_for_incomplete_chunks='all', output_final_state=True,
                               decay_for_non_mamba_blocks=True, nats_block_size=w["block"])
    else:
        mixed.mixed_attn_gdn(q, k, v, q, k, v, None, g, beta, ty, ops_for_incomplete_chunks='all', output_final_state=True,
                             decay_for_non_gdn_blocks=True, nats_block_size=w["block"])
    dt = time.perf_counter() - t0
    tok_s = Bs * w["T"] / dt * (H / w["H"])
    sample = (f"{Bs} of {w['B']} sequences, {H} of {w['H']} heads, full T={w['T']}; {dt:.1f} s of the fp32 torch-CPU oracle, "
              f"tokens/s scaled by heads")
    return dict(value=tok_s, unit="tokens/s", cores=threads, kind="port", sample=sample)


def bench_decode(args):
    """One decode step (new token of every sequence): masked attention over the cached keys/values + the gated
    delta rule on the cached state.  HBM-bound: the states are read and written once, the caches read once."""
    import torch
    from neuralattentionsearchlinear_amd import _capi
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import nats_mixed_attn_gdn_recurrent
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    _capi.lib()
    w = DECODE_WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    B, H, K, V, block = w["B"], w["H"], w["K"], w["V"], w["block"]
    TK = int(w["ctx"] * w["p_attn"]) // block * block + w["n_in_block"] + 1      # cached attention blocks + current block + new token
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    q, k, v = rn(B, 1, H, K).bfloat16(), rn(B, 1, H, K).bfloat16(), rn(B, 1, H, V).bfloat16()
    ka, va = rn(B, TK, H, K).bfloat16(), rn(B, TK, H, V).bfloat16()
    mask = torch.ones(B, H, 1, TK, dtype=torch.bool, device=dev)
    S, S0 = rn(B, H, K, V) * 0.1, rn(B, H, K, V) * 0.1
    gl = -torch.nn.functional.softplus(rn(B, 1, H))
    gcum = -torch.rand(B, H, device=dev, generator=g) * 5
    beta = torch.sigmoid(rn(B, 1, H)).bfloat16()
    ty = torch.ones(B, 1, H, 2, device=dev, dtype=torch.bfloat16)

    def step():
        return nats_mixed_attn_gdn_recurrent(q, ka, va, q, k, v, mask, S, S0, gl, gcum, beta, ty, n_tokens_in_current_block=w["n_in_block"],
                                             nats_block_size=block, ops_for_incomplete_chunks="all", decay_for_non_gdn_blocks=True)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    nbytes = B * H * K * V * 4 * 3 + B * TK * H * (K + V) * 2 + B * H * (2 * K + 2 * V) * 2 * 2
    print(json.dumps(dict(
        metric="hybrid-layer decode tokens/sec (one new token per sequence) @ctx=8192,H=16,d=128 bf16", value=B / (ms * 1e-3),
        unit="tokens/s", n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=ms, higher_is_better=True, scaling="weak",
        vs_baseline=None, dtype="bf16", data="synthetic", config=dict(workload=args.workload, **w, cached_keys=TK),
        roofline=dict(bound="hbm", kernel="gdn_recurrent_kernel+attn_masked_kernel", achieved=nbytes / (ms * 1e-3) / 1e9,
                      peak=PEAK_HBM_GBS, unit="GB/s", frac=nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, traffic=None,
                      algorithmic_bytes=nbytes, note="whole step incl. launch overheads of two kernels"))))


def bench_kv_compact(args):
    """The K/V hand-off of one prefill into the generation cache: gather the attention-typed blocks of every
    (sequence, head) into a buffer sized for them.  Pure byte movement: kept bytes read once and written once."""
    import torch
    from neuralattentionsearchlinear_amd import _capi
    from neuralattentionsearchlinear_amd.cache import NAtSLayerCache
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    _capi.lib()
    w = CACHE_WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    B, T, H, K, V, block = w["B"], w["T"], w["H"], w["K"], w["V"], w["block"]
    g = torch.Generator(device=dev).manual_seed(0)
    k = torch.randn(B, T, H, K, device=dev, generator=g).bfloat16()
    v = torch.randn(B, T, H, V, device=dev, generator=g).bfloat16()
    attn = (torch.rand(B, T // block, H, device=dev, generator=g) < w["p_attn"]).float()
    types = torch.stack([attn, 1 - attn], -1).bfloat16()
    kept = int(attn.sum())
    nbytes = 2 * kept * block * (K + V) * 2                    # kept blocks read once and written once
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    times = []
    for i in range(args.warmup + args.steps):
        cache = NAtSLayerCache(nats_block_size=block, op_for_incomplete_chunk="all")
        cache.update_attn_cache((k, v), types)
        cache._compact(types, (k, v), T // block, 0)           # allocates the cache, then one kernel launch: warm the allocator first
        torch.cuda.synchronize()
        dst_k, dst_v = cache.attn_k, cache.attn_v
        ev[0].record()
        rc = _capi.lib().natsl_kv_compact(_capi.ptr(k), _capi.ptr(v), T, 0, _capi.ptr(dst_k), _capi.ptr(dst_v), dst_k.shape[1],
                                          _capi.ptr(types), _capi.BF16, None, B, H, H, K, V, _capi.BF16, block, T // block,
                                          T // block, -1, 0, _capi.stream_ptr(dev))
        ev[1].record()
        _capi.check(rc, "natsl_kv_compact")
        torch.cuda.synchronize()
        if i >= args.warmup:
            times.append(ev[0].elapsed_time(ev[1]))
    ms = sum(times) / len(times)
    print(json.dumps(dict(
        metric="prefill K/V hand-off into the generation cache, tokens/sec @T=8192,H=16,d=128 bf16", value=B * T / (ms * 1e-3),
        unit="tokens/s", n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=ms, higher_is_better=True, scaling="weak",
        vs_baseline=None, dtype="u8", data="synthetic", config=dict(workload=args.workload, **w, kept_blocks=kept,
                                                                   cache_tokens=int(dst_k.shape[1])),
        roofline=dict(bound="hbm", kernel="kv_compact_kernel", achieved=nbytes / (ms * 1e-3) / 1e9, peak=PEAK_HBM_GBS, unit="GB/s",
                      frac=nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, traffic=None, algorithmic_bytes=nbytes, launch_ms=ms))))


def bench_softmax_bwd(args):
    """Backward of the softmax branch: dq, dk, dv and the selector's gradient from (q, k, v, o, lse, do).  Five products
    per (query, visible key) pair -- S, dP, dV, dK, dQ -- so 2.5x the forward's FLOPs; the two kernels form S and dP
    twice (once per kernel), which is not counted."""
    import torch
    from neuralattentionsearchlinear_amd import _capi, nats_util
    from neuralattentionsearchlinear_amd.attns import parallel_attn_nats_bwd, parallel_attn_nats_fwd
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    _capi.lib()
    w = BACKWARD_WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    host, d = make_inputs(w, torch, dev)
    ty, nb = nats_util.hard_select(d["logits"], force_last_block=True)
    r = nats_util.route(ty, w["T"], w["block"])
    scale = w["K"] ** -0.5
    o, lse, _ = parallel_attn_nats_fwd(d["q"], d["k"], d["v"], ty, r["nats_block_indices"], None, scale, w["block"],
                                       compute_incomplete_chunk_scores=True, n_nats_blocks=r["n_nats_blocks"])
    do = torch.randn(o.shape, device=dev, generator=torch.Generator(device=dev).manual_seed(1)).bfloat16()

    def step():
        return parallel_attn_nats_bwd(d["q"], d["k"], d["v"], o, ty, r["nats_block_indices"], r["n_nats_blocks"], None, lse, do,
                                      scale=scale, NAtS_block_size=w["block"], compute_incomplete_chunk_scores=True)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    flops = 2.5 * softmax_flops(ty.cpu(), w["T"], w["block"], w["K"], w["V"])
    print(json.dumps(dict(
        metric="softmax-branch backward tokens/sec @T=8192,H=16,d=128 bf16", value=w["B"] * w["T"] / (ms * 1e-3), unit="tokens/s",
        n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=ms, higher_is_better=True, scaling="weak", vs_baseline=None,
        dtype="bf16", data="synthetic", config=dict(workload=args.workload, **w),
        roofline=dict(bound="mfma", kernel="dq_kernel+dkdv_kernel", achieved=flops / (ms * 1e-3) / 1e12, peak=PEAK_BF16_MFMA_TFLOPS,
                      unit="TFLOP/s", frac=flops / (ms * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS, traffic=None, algorithmic_flops=flops,
                      note="whole step: delta, dq and dk/dv kernels"))))


def bench_linear_bwd(args):
    """Backward of the Gated DeltaNet branch: dq, dk, dv, dg, dbeta and the selector's gradient from (q, k, v, g, beta, do):
    the forward once more (storing every chunk's state and v_new), the reverse scan, the per-chunk gradient kernel.
    HBM-bound by design: the compulsory bytes are the six inputs and five outputs once."""
    import torch
    from neuralattentionsearchlinear_amd import _capi, nats_util
    from neuralattentionsearchlinear_amd._linear_bwd import linear_chunk_backward_hip
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    _capi.lib()
    w = LINEAR_BACKWARD_WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    host, d = make_inputs(w, torch, dev)
    ty, nb = nats_util.hard_select(d["logits"], force_last_block=True)
    do = torch.randn(d["v"].shape, device=dev, generator=torch.Generator(device=dev).manual_seed(1)).bfloat16()

    is_mamba = w.get("kind") == "mamba"

    def step():
        if is_mamba:
            return linear_chunk_backward_hip('mamba', d["q"], d["k"], d["v_l"], d["g"], None, None, ty, 1.0, w["block"], True, False, True, do,
                                             None, False)
        return linear_chunk_backward_hip('gdn', d["q"], d["k"], d["v"], d["g"], d["beta"], None, ty, w["K"] ** -0.5, w["block"], True, True,
                                         True, do, None, False)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    n_tok = w["B"] * w["T"] * w["H"]
    nbytes = n_tok * (2 * (4 * w["K"] + 3 * w["V"]) + 4 * 2 + (0 if is_mamba else 2 * 2))     # q, k, dq, dk; v, do, dv; g, dg (f32); beta, dbeta
    print(json.dumps(dict(
        metric=("Mamba2-SSD" if is_mamba else "GDN") + "-branch backward tokens/sec bf16", value=w["B"] * w["T"] / (ms * 1e-3), unit="tokens/s",
        n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=ms, higher_is_better=True, scaling="weak", vs_baseline=None,
        dtype="bf16", data="synthetic", config=dict(workload=args.workload, **w),
        roofline=dict(bound="hbm", kernel=("mamba_scale" if is_mamba else "linear_prep") + "+linear_scan+linear_bwd_scan+linear_bwd_chunk", achieved=nbytes / (ms * 1e-3) / 1e9,
                      peak=PEAK_HBM_GBS, unit="GB/s", frac=nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, traffic=None, algorithmic_bytes=nbytes,
                      note="whole step incl. the forward re-run and the host-side glue"))))


def bench_layer(args):
    """NeuralAttentionSearchLinearAttnGDN (random weights, the selector free to choose) on random hidden states: the
    projections are torch GEMMs, everything else this package's kernels.  'train' = forward + backward of a scalar loss."""
    import torch
    from neuralattentionsearchlinear_amd import _capi
    from neuralattentionsearchlinear_amd import _mixed_common
    from neuralattentionsearchlinear_amd.natsl_attn_gdn import NeuralAttentionSearchLinearAttnGDN
    _mixed_common.SAVE_CHUNK_STATES = dict(auto=None, on=True, off=False)[args.save_chunk_states]
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    _capi.lib()
    w = LAYER_WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    layer = NeuralAttentionSearchLinearAttnGDN(hidden_size=1024, expand_v=2, head_dim=128, num_heads=6, num_attn_heads=12, nats_block_size=64,
                                               ops_for_incomplete_chunks='all', decay_for_non_gdn_blocks=True, norm_eps=1e-6)
    layer = layer.to(dev).to(torch.bfloat16)
    layer.train(w["train"])
    x = torch.randn(w["B"], w["T"], 1024, device=dev).bfloat16().requires_grad_(w["train"])

    def step():
        if w["train"]:
            layer(x)[0].float().pow(2).mean().backward()
        else:
            with torch.no_grad():
                layer(x)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    print(json.dumps(dict(
        metric="GDN layer (340M geometry) " + ("training step" if w["train"] else "forward") + " tokens/sec bf16", value=w["B"] * w["T"] / (ms * 1e-3),
        unit="tokens/s", n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=ms, higher_is_better=True, scaling="weak",
        vs_baseline=None, dtype="bf16", data="synthetic", config=dict(workload=args.workload, save_chunk_states=args.save_chunk_states, **w))))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--save-chunk-states", choices=["auto", "on", "off"], default="auto",
                    help="layer workloads: what the differentiable operator keeps for the linear backward (_mixed_common.SAVE_CHUNK_STATES)")
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="hybrid_gdn_B8_T8192_H16_d128_p25", choices=sorted(WORKLOADS) + sorted(DECODE_WORKLOADS) + sorted(CACHE_WORKLOADS) + sorted(BACKWARD_WORKLOADS) + sorted(LINEAR_BACKWARD_WORKLOADS) + sorted(LAYER_WORKLOADS))
    ap.add_argument("--prewarm-ms", type=float, default=300.0,
                    help="milliseconds of untimed load before the warm-up steps, to let the GPU clocks settle (0 = none)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-heads", type=int, default=16, help="heads of the slice timed on the CPU")
    ap.add_argument("--cpu-batch", type=int, default=8, help="sequences of the slice timed on the CPU")
    ap.add_argument("--serial-branches", action="store_true",
                    help="force the softmax and the linear branch onto one stream, one after the other (default: the operator decides)")
    ap.add_argument("--concurrent-branches", action="store_true", help="force the softmax branch onto a side stream")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 1 GiB device copy after the timed steps, so that a counter run of this "
                         "command holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path shards over (batch, head) with no communication and every box has one "
              "GPU; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.workload in DECODE_WORKLOADS:
        return bench_decode(args)
    if args.workload in CACHE_WORKLOADS:
        return bench_kv_compact(args)
    if args.workload in BACKWARD_WORKLOADS:
        return bench_softmax_bwd(args)
    if args.workload in LINEAR_BACKWARD_WORKLOADS:
        return bench_linear_bwd(args)
    if args.workload in LAYER_WORKLOADS:
        return bench_layer(args)
    import torch
    from neuralattentionsearchlinear_amd import _capi, _mixed_common, nats_util
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import nats_mixed_attn_gdn
    from neuralattentionsearchlinear_amd.mixed_attn_mamba import nats_mixed_attn_mamba
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    _capi.lib()
    device = torch.device("cuda:0")
    w = WORKLOADS[args.workload]
    is_mamba = w.get("kind") == "mamba"
    host, dev = make_inputs(w, torch, device)

    events = []

    def hook(name, stream):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(stream)
        events.append((name, ev))

    def step():
        ty, nb = nats_util.hard_select(dev["logits"], force_last_block=True)
        if is_mamba:
            return nats_mixed_attn_mamba(dev["q"], dev["k"], dev["v"], dev["q"], dev["k"], dev["v_l"], None, dev["g"], ty, nb,
                                         scale_lattn=1.0, nats_block_size=w["block"], ops_for_incomplete_chunks="all",
                                         output_final_state_mamba=True, decay_for_non_mamba_blocks=True), ty
        return nats_mixed_attn_gdn(dev["q"], dev["k"], dev["v"], dev["q"], dev["k"], dev["v"], None, dev["g"], dev["beta"], ty,
                                   nb, nats_block_size=w["block"], ops_for_incomplete_chunks="all",
                                   output_final_state_gated_delta=True, decay_for_non_gdn_blocks=True), ty

    with torch.no_grad():
        if args.serial_branches or args.concurrent_branches:
            _mixed_common.CONCURRENT_BRANCHES = bool(args.concurrent_branches)
        # The GPU leaves idle at reduced clocks and needs about 40 ms of load to settle (the first 30 steps of a cold
        # run take up to 15 % longer per kernel): load it for --prewarm-ms with the same step before the W warm-up
        # steps, so that a short run measures the steady state it would also reach after more steps.
        t_pre = time.perf_counter()
        n_pre = 0
        while (time.perf_counter() - t_pre) * 1e3 < args.prewarm_ms:
            step()
            n_pre += 1
            if n_pre % 8 == 0:
                torch.cuda.synchronize()
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        _mixed_common.TIMING_HOOK = hook
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out, ty = step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        _mixed_common.TIMING_HOOK = None
        if args.calibrate_copy:
            src = torch.empty(1 << 28, dtype=torch.float32, device=device).normal_()
            dst = torch.empty_like(src)
            dst.copy_(src)  # 1 GiB read + 1 GiB written
            torch.cuda.synchronize()
            del src, dst

    ms_per_step = (t1 - t0) * 1e3 / args.steps
    n_timed_events = len(events)
    # a few more steps with the two branches one after the other on one stream: each kernel's duration alone
    with torch.no_grad():
        _mixed_common.CONCURRENT_BRANCHES = False
        step()
        torch.cuda.synchronize()
        _mixed_common.TIMING_HOOK = hook
        for _ in range(5):
            step()
        torch.cuda.synchronize()
        _mixed_common.TIMING_HOOK = None
        _mixed_common.CONCURRENT_BRANCHES = None
    tokens = w["B"] * w["T"]
    value = tokens / (ms_per_step * 1e-3)

    def avg_ms(tag, evs):
        starts = [e for n, e in evs if n == tag + ":start"]
        ends = [e for n, e in evs if n == tag + ":end"]
        return sum(s.elapsed_time(e) for s, e in zip(starts, ends)) / max(1, len(starts))

    sm_ms, lin_ms = avg_ms("softmax", events[:n_timed_events]), avg_ms("linear", events[:n_timed_events])
    sm_alone_ms, lin_alone_ms = avg_ms("softmax", events[n_timed_events:]), avg_ms("linear", events[n_timed_events:])
    types_host = ty.cpu()
    f_attn = softmax_flops(types_host, w["T"], w["block"], w["K"], w["V"])
    f_gdn = (mamba_flops if is_mamba else gdn_flops)(types_host, w["K"], w["V"], per_block=w["block"] // 64)
    B, T, H, K, V = w["B"], w["T"], w["H"], w["K"], w["V"]
    traffic, traffic_source = measured_traffic(args.workload)
    # the linear branch (prep + scan kernels): algorithmic bytes = q, k, v read once, o written once, g and beta, final state
    # (the Mamba workload's B and C are stored per head here, as the operator takes them, and counted so)
    lin_bytes = B * T * H * (2 * K + 2 * V) * 2 + B * T * H * (4 if is_mamba else 6) + B * H * K * V * 4
    roof_lin = dict(bound="hbm", kernel=("mamba_scale_kernel" if is_mamba else "linear_prep_kernel") + "+linear_scan_kernel", achieved=lin_bytes / (lin_ms * 1e-3) / 1e9,
                    peak=PEAK_HBM_GBS, unit="GB/s", frac=lin_bytes / (lin_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                    traffic=(traffic or {}).get("linear_bytes"), launch_ms=lin_ms, algorithmic_bytes=lin_bytes,
                    algorithmic_flops=f_gdn, frac_of_mfma_peak=f_gdn / (lin_ms * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                    launch_ms_alone=lin_alone_ms)
    if f_attn >= f_gdn:
        achieved = f_attn / (sm_ms * 1e-3) / 1e12
        roof = dict(bound="mfma", kernel=softmax_kernel_name(B, T, H, w["block"]), achieved=achieved, peak=PEAK_BF16_MFMA_TFLOPS,
                    unit="TFLOP/s", frac=achieved / PEAK_BF16_MFMA_TFLOPS, traffic=(traffic or {}).get("softmax_bytes"),
                    traffic_source=traffic_source, launch_ms=sm_ms, algorithmic_flops=f_attn,
                    # the same kernel with the GPU to itself (branches launched one after the other, outside the timed region)
                    launch_ms_alone=sm_alone_ms, frac_alone=f_attn / (sm_alone_ms * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS)
    else:
        # GDN-only workload: HBM-bound
        roof = dict(roof_lin, traffic_source=traffic_source)
    probe = clock_probe(torch, device)

    rec = dict(
        metric="hybrid-layer fwd tokens/sec @T=8192,H=16,d=128 bf16; % of MFMA/HBM roofline",
        value=value, unit="tokens/s", n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=ms_per_step,
        higher_is_better=True, scaling="weak", vs_baseline=None, dtype="bf16", data="synthetic",
        config=dict(workload=args.workload, **w, attn_fraction=float(types_host[..., 0].float().mean()),
                    softmax_ms=sm_ms, linear_ms=lin_ms, softmax_alone_ms=sm_alone_ms, linear_alone_ms=lin_alone_ms, step_flops=f_attn + f_gdn,
                    step_frac_of_mfma_peak=(f_attn + f_gdn) / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS),
        roofline=roof,
        roofline_linear=roof_lin,
        clock=probe,
        prewarm=dict(ms=args.prewarm_ms, steps=n_pre),
    )
    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline(host, w, types_host, torch, max_heads=args.cpu_heads, max_batch=args.cpu_batch)
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
