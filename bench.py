"""Benchmark of the fused-attention hot path on one MI355X.

A step is one call of the prefill operator on the Llama-3-8B-shaped workload (B=1, Hq=32, Hkv=8,
S=4096, D=128, fp16, causal dense mask); `value` is its throughput in algorithmic TFLOP/s
(4*D*Hq*attended pairs), inputs resident in HBM, every kernel the op launches inside the timed
region.  The decode workload (B=64, ctx in [512,8192]) is timed in the same run and reported
under "decode" with its own HBM roofline (and again over Q8_0 caches under "decode_q8_0"), the steps that feed
attention under "rope", "rope_kv_append" (into Q8_0 caches: "rope_kv_append_q8_0"; with the per-head q/k norm: "rope_kv_append_norm"),
"rmsnorm", "gemm", "qkv" and "gemm_q8_0" (a decode step's projection against a weight of Q8_0 blocks), and the
reference's CPU attention path (torch SDPA in fp32 on the host cores) under "cpu_baseline".  Prints ONE JSON line.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "minfer-python_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)
sys.path.append(os.path.join(PKG, "apps"))   # last: its profile.py must not shadow the standard library's

PEAK_MFMA_TFLOPS = 2500.0   # MI355X dense fp16/bf16
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each scaled by what the
# same counter reads for a 1 GiB copy: x2.0 and x1.0), classify+main and split+combine respectively
# These are figures from those earlier counter runs, not measured in the run that prints them.
TRAFFIC_SOURCE = "profiles/hbm_traffic_all_kernels_pmc.md (rocprofv3 --pmc runs of the same workloads; not re-measured by this run)"
PREFILL_TRAFFIC_BYTES = 107080 * 1024
DECODE_TRAFFIC_BYTES = 1092850 * 1024
ROPE_TRAFFIC_BYTES = 393314 * 1024          # il_rope on [8,4096,48,128], rotary 64
APPEND_TRAFFIC_BYTES = 786532 * 1024        # rope_kv_append, B=8 L=4096 Llama-3-8B heads
NORM_TRAFFIC_BYTES = 786691 * 1024          # rmsnorm on [8,4096,6144]
GEMM_TRAFFIC_BYTES = 229729 * 1024          # gemm 4096^3 (A and B panels are re-read by several XCDs)
DECODE_Q8_TRAFFIC_BYTES = 598274 * 1024     # decode over Q8_0 caches (split + combine)
APPEND_Q8_TRAFFIC_BYTES = 737591 * 1024     # rope_kv_append into Q8_0 caches
APPEND_NORM_TRAFFIC_BYTES = 786609 * 1024   # rope_kv_append_norm, the same shape
QKV_TRAFFIC_BYTES = 377962 * 1024           # qkv in one launch, M=K=4096, N=4096+1024+1024
LONG_TRAFFIC_BYTES = 2721732 * 1024         # long-context prefill (classify + main), S=32768 bf16: the 1 GiB mask once, K/V re-fetched past the 4 MiB L2s
RAGGED_TRAFFIC_BYTES = 747982 * 1024        # packed ragged prefill (T=20514, Hq=64)
GEMM_Q8_TRAFFIC_BYTES = 61124 * 1024        # one token against a 14336 x 4096 weight of Q8_0 blocks
GEMM_DECODE_TRAFFIC_BYTES = 120705 * 1024   # 64 tokens against the same weight in fp16, [N, K]
# The kernel sources the counter runs were made against (first 12 hex digits of each file's sha1).  A row one of whose
# sources has changed since carries "traffic_stale": true, so a constant that describes an earlier kernel says so.
TRAFFIC_MEASURED_AGAINST = {
    "attn_common.h": "4dea1f54fd55",
    "attn_prefill.hip": "d7de40fffd05",
    "attn_decode.hip": "af41b9ac94d8",
    "quant_q8.h": "4fea6a94e300",
    "rope.hip": "b4fd0618b44e",
    "rmsnorm.hip": "f6c4e575f461",
    "gemm.hip": "89047d798694",
}
TRAFFIC_ROW_SOURCES = {
    "": ("attn_common.h", "attn_prefill.hip"), "long_context": ("attn_common.h", "attn_prefill.hip"), "ragged": ("attn_common.h", "attn_prefill.hip"),
    "decode": ("attn_common.h", "attn_decode.hip"), "decode_q8_0": ("attn_common.h", "attn_decode.hip", "quant_q8.h"),
    "rope": ("attn_common.h", "rope.hip"), "rope_kv_append": ("attn_common.h", "rope.hip"),
    "rope_kv_append_q8_0": ("attn_common.h", "rope.hip", "quant_q8.h"), "rope_kv_append_norm": ("attn_common.h", "rope.hip"),
    "rmsnorm": ("attn_common.h", "rmsnorm.hip"), "gemm": ("attn_common.h", "gemm.hip"), "qkv": ("attn_common.h", "gemm.hip"),
    "gemm_q8_0": ("attn_common.h", "gemm.hip", "quant_q8.h"), "gemm_decode": ("attn_common.h", "gemm.hip"),
}


def source_digest(name):
    import hashlib
    with open(os.path.join(PKG, "csrc", name), "rb") as f:
        return hashlib.sha1(f.read()).hexdigest()[:12]


def mark_stale_traffic(rec):
    """Adds "traffic_stale" to every roofline that quotes a traffic constant."""
    changed = {n for n, d in TRAFFIC_MEASURED_AGAINST.items() if source_digest(n) != d}
    for row, sources in TRAFFIC_ROW_SOURCES.items():
        roof = (rec if row == "" else rec[row]).get("roofline", {})
        if roof.get("traffic") is not None:
            roof["traffic_stale"] = bool(changed.intersection(sources))


class HipEvents:
    """hipEvent timing on an explicit stream through libamdhip64 (the kernels are launched on the
    stream handed to the op, which is torch's current stream)."""

    def __init__(self):
        import torch
        self.hip = ctypes.CDLL(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [ctypes.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]

    def event(self):
        e = ctypes.c_void_p()
        assert self.hip.hipEventCreate(ctypes.byref(e)) == 0
        return e

    def time_region(self, fn, stream, n):
        """Average duration (ms) of n back-to-back calls of fn bracketed by ONE pair of events on `stream`: what the
        GPU needs per call when calls follow each other, launch gaps included, no host clock involved."""
        a, b = self.event(), self.event()
        assert self.hip.hipEventRecord(a, stream) == 0
        for _ in range(n):
            fn()
        assert self.hip.hipEventRecord(b, stream) == 0
        assert self.hip.hipEventSynchronize(b) == 0
        t = ctypes.c_float()
        assert self.hip.hipEventElapsedTime(ctypes.byref(t), a, b) == 0
        return t.value / n

    def time_each(self, fn, stream, n):
        """Average and median duration (ms) of n calls of fn, each bracketed by events on `stream`."""
        pairs = [(self.event(), self.event()) for _ in range(n)]
        for a, b in pairs:
            assert self.hip.hipEventRecord(a, stream) == 0
            fn()
            assert self.hip.hipEventRecord(b, stream) == 0
        ms = []
        for a, b in pairs:
            assert self.hip.hipEventSynchronize(b) == 0
            t = ctypes.c_float()
            assert self.hip.hipEventElapsedTime(ctypes.byref(t), a, b) == 0
            ms.append(t.value)
        ms_sorted = sorted(ms)
        return sum(ms) / len(ms), ms_sorted[len(ms) // 2]


def _median3(fn):
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[1]


def cpu_baseline(torch, workloads, refs, L):
    """The reference's CPU attention path: refs.flash_attn = torch SDPA, fp32, K/V pre-expanded outside
    the timed region, on the same seeded inputs up-cast (reference: apps/benchmark.py:240-248)."""
    q, k, v, mask = workloads.llama8b_prefill(seed=0, L=L)
    q, k, v = q.float(), k.float().repeat_interleave(4, 1), v.float().repeat_interleave(4, 1)
    refs.flash_attn(q[:, :4], k[:, :4], v[:, :4], mask)  # warm-up on a slice
    t = _median3(lambda: refs.flash_attn(q, k, v, mask))
    flops = workloads.prefill_flops(32, 128, [L])
    return {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"refs.flash_attn (torch SDPA, fp32, dense causal mask) on the full S={L} workload, median of 3: {t * 1e3:.1f} ms",
            "host_cpus": os.cpu_count()}


def cpu_baseline_plumbing(torch, workloads, refs):
    """BASELINE configs[0] (B=1, Hq=8, Hkv=2, S=256, D=64, fp32): the reference's CPU path on it."""
    q, k, v, mask = workloads.cpu_plumbing(seed=0)
    k, v = k.repeat_interleave(4, 1), v.repeat_interleave(4, 1)
    refs.flash_attn(q, k, v, mask)
    t = _median3(lambda: refs.flash_attn(q, k, v, mask))
    flops = workloads.prefill_flops(8, 64, [256])
    return {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"refs.flash_attn (torch SDPA, fp32) on the full B=1 Hq=8 Hkv=2 S=256 D=64 workload, median of 3: {t * 1e3:.3f} ms"}


def cpu_baseline_decode(torch, workloads, refs, n_seq=16):
    """The reference's CPU path on the decode workload: SDPA in fp32 with Lq = 1 and the [B,1,1,Lmax] mask that ctx_lens
    gives, K/V caches pre-expanded to the query heads outside the timed region.  A sample of `n_seq` of the 64
    sequences (the expanded fp32 caches of all 64 would be 17 GB); same algorithmic bytes per sequence as the GPU figure."""
    q, kc, vc, ctx = workloads.decode_cache(seed=0, B=n_seq)
    q, kc, vc = q.float(), kc.float().repeat_interleave(4, 1), vc.float().repeat_interleave(4, 1)
    refs.flash_attn_decode(q[:1], kc[:1], vc[:1], ctx[:1])
    t = _median3(lambda: refs.flash_attn_decode(q, kc, vc, ctx))
    nbytes = workloads.decode_bytes(ctx.tolist(), 32, 8, 128)
    return {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"refs.flash_attn_decode (torch SDPA, fp32, mask from ctx_lens) on {n_seq} of the 64 sequences "
                      f"(sum ctx = {int(ctx.sum())} rows, fp16-cache algorithmic bytes), median of 3: {t * 1e3:.1f} ms"}


def cpu_baseline_ragged(torch, workloads, refs):
    """The reference's CPU path on the packed workload: one refs.flash_attn call per sequence with its causal bool mask
    (masks and the GQA expansion built outside the timed region), times summed over the 16 sequences."""
    q, k, v, cu = workloads.ragged_prefill(seed=0)
    n_rep = q.shape[1] // k.shape[1]
    q, k, v = q.float(), k.float().repeat_interleave(n_rep, 1), v.float().repeat_interleave(n_rep, 1)
    cu = cu.tolist()
    parts = [(q[:, :, lo:hi], k[:, :, lo:hi], v[:, :, lo:hi], workloads.causal_mask(1, hi - lo)) for lo, hi in zip(cu[:-1], cu[1:])]
    refs.flash_attn(*parts[0])

    def run():
        for a in parts:
            refs.flash_attn(*a)
    t = _median3(run)
    lens = [hi - lo for lo, hi in zip(cu[:-1], cu[1:])]
    flops = workloads.prefill_flops(q.shape[1], 128, lens)
    return {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"refs.flash_attn (torch SDPA, fp32, causal bool mask) once per sequence on the full packed workload "
                      f"(16 sequences, T={cu[-1]}), summed, median of 3: {t * 1e3:.1f} ms"}


def cpu_baseline_long(torch, workloads, refs, L=32768, rows=1024, cap_s=60.0):
    """The reference's CPU path on the long-context workload, bounded: the last `rows` query rows of the S=32768 problem
    against all keys (SDPA, fp32, their rows of the dense causal mask), one timed run; the whole problem is 32 times
    that.  Reported as capped if the run exceeds `cap_s`."""
    g = torch.Generator().manual_seed(0)
    q = (0.5 * torch.randn(1, 32, rows, 128, generator=g)).bfloat16().float()
    k = (0.5 * torch.randn(1, 8, L, 128, generator=g)).bfloat16().float().repeat_interleave(4, 1)
    v = (0.5 * torch.randn(1, 8, L, 128, generator=g)).bfloat16().float().repeat_interleave(4, 1)
    i = torch.arange(L - rows, L)
    mask = (torch.arange(L)[None, :] <= i[:, None])[None, None].contiguous()
    refs.flash_attn(q[:, :1, :64], k[:, :1], v[:, :1], mask[:, :, :64])
    t0 = time.perf_counter()
    refs.flash_attn(q, k, v, mask)
    t = time.perf_counter() - t0
    flops = 4.0 * 128 * 32 * sum(range(L - rows + 1, L + 1))
    return {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port", "capped": t > cap_s,
            "sample": f"refs.flash_attn (torch SDPA, fp32) on the last {rows} query rows of the S={L} workload against all keys "
                      f"({flops:.3e} of its 8.796e12 algorithmic flop), one run: {t * 1e3:.1f} ms"}


def rope_cpu_baseline(torch, workloads, refs):
    """The reference's CPU statement of il_rope (torch expressions in fp32; reference: refs.py:12-29) on one
    batch entry of the reference test's shape."""
    x = workloads.rope_input(seed=0, B=1)
    refs.il_rope(x[:, :64], 64, 2048, 1e6)
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        refs.il_rope(x, 64, 2048, 1e6)
        ts.append(time.perf_counter() - t0)
    t = sorted(ts)[1]
    return {"value": workloads.rope_bytes(1, 4096, 48, 64) / t / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"refs.il_rope (torch, fp32) on x [1,4096,48,128], median of 3: {t * 1e3:.1f} ms"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=300,
                    help="untimed steps right before the timed ones (a time-based pre-warm of the clocks runs before them in any case)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph", action="store_true", help="replay one captured HIP graph per step instead of launching from Python")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the attention path shards by batch / KV head without any "
                 "exchange, and this build has no multi-GPU launcher. Run with --gpus 1.")

    import torch
    import workloads
    from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType
    from minfer.kernels import KernelBackend, refs

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: the operators have no CPU implementation")
    kerns = KernelBackend("torch_ext")
    dev = "cuda:0"
    torch.cuda.set_device(0)
    qt = GGMLQuantizationType.F16
    qb, qs = GGML_QUANT_SIZES[qt]
    ev = HipEvents()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    # ---- prefill: the step -----------------------------------------------------------------
    L = 4096
    q, k, v, mask = workloads.llama8b_prefill(seed=0, device=dev, L=L)
    out = torch.zeros_like(q)
    eager_step = lambda: kerns.flash_attn(qt, qb, qs, q, k, v, mask, out)
    eager_step()
    torch.cuda.synchronize()
    if not args.graph:
        step = eager_step
    else:
        # One step (mask classification + attention kernel) captured once and replayed: the timed loop then
        # measures the GPU, not the Python/dispatcher launch path.  The op records no memset nodes.
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            eager_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            eager_step()
        step = graph.replay
        ref_out = out.clone()
        out.zero_()
        step()
        torch.cuda.synchronize()
        assert torch.equal(out, ref_out), "graph replay differs from the eager result"
    # The chip needs some 15 ms of continuous work after an idle period to reach its clocks (a loop started cold
    # averages 174 us per call instead of 146): whatever --warmup says, the step first runs back to back until
    # PREWARM_MS of GPU time have passed, so that a short run (--warmup 5 --steps 20) measures the same steady
    # state as a long one.
    PREWARM_MS = 100.0
    prewarm_ms, prewarm_calls = 0.0, 0
    while prewarm_ms < PREWARM_MS:
        prewarm_ms += ev.time_region(step, stream, 50) * 50
        prewarm_calls += 50
    for _ in range(args.warmup):
        step()
    # the timed region: exactly --steps steps, by the host clock between two synchronisations and, over the same
    # steps, by one pair of events on the launch stream
    t_a, t_b = ev.event(), ev.event()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    assert ev.hip.hipEventRecord(t_a, stream) == 0
    for _ in range(args.steps):
        step()
    assert ev.hip.hipEventRecord(t_b, stream) == 0
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    t_el = ctypes.c_float()
    assert ev.hip.hipEventElapsedTime(ctypes.byref(t_el), t_a, t_b) == 0
    region_ms = t_el.value / args.steps
    # a region of at least 200 steps for the roofline figure when --steps is smaller (the same region otherwise)
    event_steps = max(args.steps, 200)
    avg_ms = region_ms if event_steps == args.steps else ev.time_region(step, stream, event_steps)
    _, med_ms = ev.time_each(step, stream, min(event_steps, 200))
    flops = workloads.prefill_flops(32, 128, [L])
    tflops = flops / (wall_ms * 1e-3) / 1e12
    achieved = flops / (avg_ms * 1e-3) / 1e12

    # ---- decode ------------------------------------------------------------------------------
    qd, kc, vc, ctx = workloads.decode_cache(seed=0, device=dev)
    outd = torch.zeros_like(qd)
    dstep = lambda: kerns.flash_attn_decode(qt, qb, qs, qd, kc, vc, ctx, outd)
    for _ in range(max(args.warmup, 100)):
        dstep()
    torch.cuda.synchronize()
    _, d_med_ms = ev.time_each(dstep, stream, min(max(args.steps, 20), 100))
    d_avg_ms = ev.time_region(dstep, stream, min(max(args.steps, 20), 100))
    dbytes = workloads.decode_bytes(ctx.tolist(), 32, 8, 128)
    d_gbs = dbytes / (d_avg_ms * 1e-3) / 1e9
    # the same decode over Q8_0 caches (34 bytes per 32 values), quantised on the device from the fp16 caches
    q8 = GGMLQuantizationType.Q8_0
    q8b, q8s = GGML_QUANT_SIZES[q8]
    kq8, vq8 = workloads.q8_0_rows(kc), workloads.q8_0_rows(vc)
    del kc, vc
    d8step = lambda: kerns.flash_attn_decode(q8, q8b, q8s, qd, kq8, vq8, ctx, outd)
    for _ in range(max(args.warmup, 100)):
        d8step()
    torch.cuda.synchronize()
    _, d8_med_ms = ev.time_each(d8step, stream, min(max(args.steps, 20), 100))
    d8_avg_ms = ev.time_region(d8step, stream, min(max(args.steps, 20), 100))
    d8bytes = workloads.decode_bytes_q8_0(ctx.tolist(), 32, 8, 128)
    d8_gbs = d8bytes / (d8_avg_ms * 1e-3) / 1e9
    del kq8, vq8

    # ---- the two other prefill configurations: long context (bf16) and ragged packed sequences ----
    lq, lk, lv, lmask = workloads.long_context_prefill(seed=0, device=dev)
    lout = torch.empty_like(lq)
    bt = GGMLQuantizationType.BF16
    btb, bts = GGML_QUANT_SIZES[bt]
    lstep = lambda: kerns.flash_attn(bt, btb, bts, lq, lk, lv, lmask, lout)
    for _ in range(5):
        lstep()
    torch.cuda.synchronize()
    _, l_med_ms = ev.time_each(lstep, stream, 10)
    l_avg_ms = ev.time_region(lstep, stream, 10)
    lflops = workloads.prefill_flops(32, 128, [lq.shape[2]])
    l_tf = lflops / (l_avg_ms * 1e-3) / 1e12
    del lq, lk, lv, lmask, lout
    vq, vk, vv, vcu = workloads.ragged_prefill(seed=0, device=dev)
    vlens = (vcu[1:] - vcu[:-1]).tolist()
    vout = torch.empty_like(vq)
    vstep = lambda: kerns.flash_attn_varlen(qt, qb, qs, vq, vk, vv, vcu, max(vlens), vout)
    for _ in range(50):
        vstep()
    torch.cuda.synchronize()
    _, v_med_ms = ev.time_each(vstep, stream, 50)
    v_avg_ms = ev.time_region(vstep, stream, 50)
    vflops = workloads.prefill_flops(64, 128, vlens)
    v_tf = vflops / (v_avg_ms * 1e-3) / 1e12
    del vq, vk, vv, vout

    # ---- the step before attention: rotary embedding, alone and fused with the cache append ----
    x = workloads.rope_input(seed=0, device=dev)                      # the reference test's shape
    rstep = lambda: kerns.il_rope(64, 2048, 1e6, x)
    for _ in range(200):
        rstep()
    torch.cuda.synchronize()
    _, r_med_ms = ev.time_each(rstep, stream, 50)
    r_avg_ms = ev.time_region(rstep, stream, 50)
    rbytes = workloads.rope_bytes(8, 4096, 48, 64)
    r_gbs = rbytes / (r_avg_ms * 1e-3) / 1e9
    del x
    aq, ak, av, apos, akc, avc = workloads.kv_append(seed=0, device=dev, B=8, L=4096)
    astep = lambda: kerns.rope_kv_append(1, 128, 5e5, aq, ak, av, apos, akc, avc)
    for _ in range(100):
        astep()
    torch.cuda.synchronize()
    _, a_med_ms = ev.time_each(astep, stream, 50)
    a_avg_ms = ev.time_region(astep, stream, 50)
    abytes = workloads.kv_append_bytes(8, 4096, 32, 8, 128, 128)
    a_gbs = abytes / (a_avg_ms * 1e-3) / 1e9
    # the same producer with the per-head q/k RMSNorm (Qwen3/Gemma3-style) applied first, in the same launch
    wqn = torch.ones(128, dtype=torch.float16, device=dev)
    wkn = torch.ones(128, dtype=torch.float16, device=dev)
    anstep = lambda: kerns.rope_kv_append_norm(1, 128, 5e5, 1e-6, aq, ak, av, wqn, wkn, apos, akc, avc)
    for _ in range(100):
        anstep()
    torch.cuda.synchronize()
    _, an_med_ms = ev.time_each(anstep, stream, 50)
    an_avg_ms = ev.time_region(anstep, stream, 50)
    an_gbs = abytes / (an_avg_ms * 1e-3) / 1e9
    del akc, avc
    akq = torch.zeros(8, 8, 4096, 128 // 32 * 34, dtype=torch.uint8, device=dev)
    avq = torch.zeros_like(akq)
    a8step = lambda: kerns.rope_kv_append(1, 128, 5e5, aq, ak, av, apos, akq, avq)
    for _ in range(100):
        a8step()
    torch.cuda.synchronize()
    _, a8_med_ms = ev.time_each(a8step, stream, 50)
    a8_avg_ms = ev.time_region(a8step, stream, 50)
    a8bytes = workloads.kv_append_bytes_q8_0(8, 4096, 32, 8, 128, 128)
    a8_gbs = a8bytes / (a8_avg_ms * 1e-3) / 1e9
    del aq, ak, av, akq, avq
    nshape = (8, 4096, 6144)                                          # the reference test's per-token shape
    nx, nw = workloads.rmsnorm_input(nshape, seed=0, device=dev)
    nout = torch.empty_like(nx)
    nstep = lambda: kerns.rmsnorm(1e-6, nx, nw, nout)
    for _ in range(100):
        nstep()
    torch.cuda.synchronize()
    _, n_med_ms = ev.time_each(nstep, stream, 50)
    n_avg_ms = ev.time_region(nstep, stream, 50)
    nbytes = workloads.rmsnorm_bytes(nshape)
    n_gbs = nbytes / (n_avg_ms * 1e-3) / 1e9
    del nx, nout
    # ---- projection GEMM: the reference's published HGEMM size, and its QKV projection shape ---------
    ga, gw, gbias = workloads.gemm_input(4096, 4096, 4096, seed=0, device=dev)
    gout = torch.empty_like(gbias)
    gstep = lambda: kerns.gemm(qt, qb, qs, 1.0, 0.0, ga, gw, gbias, gout)
    for _ in range(100):
        gstep()
    torch.cuda.synchronize()
    _, g_med_ms = ev.time_each(gstep, stream, 50)
    g_avg_ms = ev.time_region(gstep, stream, 50)
    gflops = workloads.gemm_flops(4096, 4096, 4096)
    g_tf = gflops / (g_avg_ms * 1e-3) / 1e12
    del ga, gw, gbias, gout
    # the QKV projection of the prefill shape, three weight matrices in one launch
    px = workloads.gemm_input(4096, 4096, 4096, seed=1, device=dev)[0]
    pwq = workloads.gemm_input(4096, 4096, 4096, seed=2, device=dev)[1].t().contiguous()   # [out, hidden]
    pwk = pwq[:1024].clone()
    pwv = pwq[1024:2048].clone()
    pq = torch.empty(1, 4096, 4096, dtype=torch.float16, device=dev)
    pk = torch.empty(1, 4096, 1024, dtype=torch.float16, device=dev)
    pv = torch.empty_like(pk)
    pstep = lambda: kerns.qkv(qt, qt, qt, qb, qb, qb, qs, qs, qs, px, pwq, pwk, pwv, pq, pk, pv)
    for _ in range(100):
        pstep()
    torch.cuda.synchronize()
    _, p_med_ms = ev.time_each(pstep, stream, 50)
    p_avg_ms = ev.time_region(pstep, stream, 50)
    pflops = workloads.gemm_flops(4096, 6144, 4096)
    p_tf = pflops / (p_avg_ms * 1e-3) / 1e12
    del px, pwq, pwk, pwv, pq, pk, pv
    # A decode step's projections.  A decode step walks through the weights of every layer, far more than the 256 MB
    # last-level cache holds, so the calls here cycle over copies of the weight (640 MiB or more in all): one weight
    # called again and again would be served by that cache and run a third faster ("ms_weight_cached" beside "ms").
    def cycle(fns):
        state = [0]
        def step():
            fns[state[0] % len(fns)]()
            state[0] += 1
        return step

    # ... against a weight kept as Q8_0 blocks (Llama-3-8B FFN up: 14336 x 4096), one token
    q8 = GGMLQuantizationType.Q8_0
    q8b, q8s = GGML_QUANT_SIZES[q8]
    wf = workloads.gemm_input(16, 14336, 4096, seed=3, device=dev)[1].t().contiguous()       # [14336, 4096] fp16
    wq8 = torch.empty(14336, 4096 // 32 * 34, dtype=torch.uint8, device=dev)
    kerns._quant(q8, q8b, q8s, wf, wq8)
    del wf
    wq8s = [wq8] + [wq8.clone() for _ in range(10)]                                            # 11 x 59.5 MiB
    xa = workloads.gemm_input(1, 16, 4096, seed=4, device=dev)[0]                              # [1, 1, 4096]
    xo = torch.zeros(1, 1, 14336, dtype=torch.float16, device=dev)
    q8step = cycle([(lambda w=w: kerns.gemm(q8, q8b, q8s, 1.0, 0.0, xa, w, xo, xo)) for w in wq8s])
    q8same = lambda: kerns.gemm(q8, q8b, q8s, 1.0, 0.0, xa, wq8, xo, xo)
    for _ in range(100):
        q8step()
    torch.cuda.synchronize()
    _, q8_med_ms = ev.time_each(q8step, stream, 55)
    q8_avg_ms = ev.time_region(q8step, stream, 220)
    q8_cached_ms = ev.time_region(q8same, stream, 200)
    q8bytes = 14336 * (4096 // 32 * 34) + 4096 * 2 + 14336 * 2
    q8_gbs = q8bytes / (q8_avg_ms * 1e-3) / 1e9
    del wq8, wq8s, xa, xo

    # ... and for the decode batch of BASELINE configs[2]: 64 tokens against the fp16 weight as [N, K]
    gwn = workloads.gemm_input(16, 14336, 4096, seed=3, device=dev)[1].t().contiguous()      # [14336, 4096]
    gwns = [gwn] + [gwn.clone() for _ in range(5)]                                             # 6 x 112 MiB
    gxa = workloads.gemm_input(64, 16, 4096, seed=5, device=dev)[0]                            # [1, 64, 4096]
    gxo = torch.zeros(1, 64, 14336, dtype=torch.float16, device=dev)
    gdstep = cycle([(lambda w=w: kerns.gemm(qt, qb, qs, 1.0, 0.0, gxa, w, gxo, gxo)) for w in gwns])
    gdsame = lambda: kerns.gemm(qt, qb, qs, 1.0, 0.0, gxa, gwn, gxo, gxo)
    for _ in range(100):
        gdstep()
    torch.cuda.synchronize()
    _, gd_med_ms = ev.time_each(gdstep, stream, 54)
    gd_avg_ms = ev.time_region(gdstep, stream, 204)
    gd_cached_ms = ev.time_region(gdsame, stream, 200)
    gdbytes = 14336 * 4096 * 2 + 64 * 4096 * 2 + 64 * 14336 * 2
    gd_gbs = gdbytes / (gd_avg_ms * 1e-3) / 1e9
    del gwn, gwns, gxa, gxo

    # ---- BASELINE configs[0] (the CPU-plumbing shape: B=1, Hq=8, Hkv=2, S=256, D=64) through the GPU op; its fp32
    # inputs are rounded to fp16, the op having no fp32 form.  Two launches of a few microseconds: launch-bound.
    cq, ck, cv, cmask = workloads.cpu_plumbing(seed=0)
    cq, ck, cv, cmask = cq.half().to(dev), ck.half().to(dev), cv.half().to(dev), cmask.to(dev)
    cout = torch.empty_like(cq)
    cstep = lambda: kerns.flash_attn(qt, qb, qs, cq, ck, cv, cmask, cout)
    for _ in range(50):
        cstep()
    torch.cuda.synchronize()
    _, c_med_ms = ev.time_each(cstep, stream, 50)
    c_avg_ms = ev.time_region(cstep, stream, 50)
    cflops = workloads.prefill_flops(8, 64, [256])

    # ---- calibration: what the chip sustains on the matrix instruction alone, on operand values of the benchmarks'
    # distribution (the nominal peak assumes 2.4 GHz, which the chip does not hold with the matrix pipes busy) ----
    import calibration
    sus_f16 = calibration.mfma_rate(torch.float16, "random", timed_ms=100.0, prewarm_ms=100.0)
    sus_bf16 = calibration.mfma_rate(torch.bfloat16, "random", timed_ms=100.0, prewarm_ms=100.0)
    # ... and on the prefill kernel's own per-tile instruction mix (MFMAs + LDS fragment reads + softmax vector work) with
    # no memory traffic, barrier or bookkeeping in the loop: what an attention kernel without any fixed cost would reach
    mix_f16 = calibration.attn_mix_rate(torch.float16, "random", True, True, timed_ms=100.0, prewarm_ms=100.0)
    mix_bf16 = calibration.attn_mix_rate(torch.bfloat16, "random", True, True, timed_ms=100.0, prewarm_ms=100.0)

    def mfma_roofline(achieved_tf, sustained, mix=None, **extra):
        r = {"bound": "mfma", "achieved": achieved_tf, "peak": PEAK_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": achieved_tf / PEAK_MFMA_TFLOPS,
             "sustained_mfma_only": sustained["tflops"], "frac_of_sustained": achieved_tf / sustained["tflops"]}
        if mix is not None:
            r["sustained_attention_mix"] = mix["tflops"]
            r["frac_of_attention_mix"] = achieved_tf / mix["tflops"]
        r.update(extra)
        return r

    rec = {
        "metric": "prefill attn TFLOP/s + decode KV GB/s (Llama-3-8B GQA), % of roofline",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms, "event_ms_per_step": region_ms, "event_steps": event_steps,
        "prewarm_ms": prewarm_ms, "prewarm_calls": prewarm_calls, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic", "launch": "hipgraph replay of one op call" if args.graph else "eager",
        "ms_is": "every row's ms: back-to-back calls between ONE pair of HIP events on the op's stream, divided by the calls (a pair around "
                 "every call adds 2-3 us, a tenth of the shortest kernels here); median_ms: a pair around every call",
        "config": {"workload": "prefill B=1 Hq=32 Hkv=8 S=4096 D=128 fp16 causal dense-mask (BASELINE configs[1])",
                   "global_batch": 1, "seq_len": L, "parallelism": "single-gpu"},
        "roofline": mfma_roofline(achieved, sus_f16, mix_f16, traffic=PREFILL_TRAFFIC_BYTES, traffic_source=TRAFFIC_SOURCE,
                                  kernel="classify_mask_kernel + prefill_kernel<F16,128,dense>",
                                  algorithmic_flops=flops, avg_ms=avg_ms, median_ms=med_ms),
        "decode": {"value": d_gbs, "unit": "GB/s", "ms": d_avg_ms, "median_ms": d_med_ms,
                   "workload": "decode B=64 Hq=32 Hkv=8 D=128 fp16 ctx~U[512,8192] cache [64,8,8192,128] (BASELINE configs[2])",
                   "roofline": {"bound": "hbm", "achieved": d_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                "frac": d_gbs / PEAK_HBM_GBS, "traffic": DECODE_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE,
                                "kernel": "decode_split_kernel<F16,128> + decode_combine_kernel",
                                "algorithmic_bytes": dbytes}},
    }
    rec["decode_q8_0"] = {"value": d8_gbs, "unit": "GB/s", "ms": d8_avg_ms, "median_ms": d8_med_ms,
                          "speedup_over_fp16_cache": d_avg_ms / d8_avg_ms,
                          "workload": "the decode workload over Q8_0 caches, uint8 [64,8,8192,136] (34-byte blocks of 32 values), q/out fp16",
                          "roofline": {"bound": "hbm", "achieved": d8_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                       "frac": d8_gbs / PEAK_HBM_GBS, "traffic": DECODE_Q8_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE,
                                       "kernel": "decode_split_q8_kernel<128> + decode_combine_kernel",
                                       "algorithmic_bytes": d8bytes}}
    rec["long_context"] = {"value": l_tf, "unit": "TFLOP/s", "ms": l_avg_ms, "median_ms": l_med_ms,
                           "workload": "prefill B=1 Hq=32 Hkv=8 S=32768 D=128 bf16 causal dense-mask, mask 1 GiB (BASELINE configs[3])",
                           "roofline": mfma_roofline(l_tf, sus_bf16, mix_bf16, traffic=LONG_TRAFFIC_BYTES, traffic_source=TRAFFIC_SOURCE,
                                                     kernel="classify_mask_kernel + prefill_kernel<BF16,128,dense>", algorithmic_flops=lflops)}
    rec["ragged"] = {"value": v_tf, "unit": "TFLOP/s", "ms": v_avg_ms, "median_ms": v_med_ms,
                     "workload": f"packed prefill of 16 sequences, lengths U[128,2048] (T={sum(vlens)}), Hq=64 Hkv=8 D=128 fp16, causal within a sequence (BASELINE configs[4])",
                     "roofline": mfma_roofline(v_tf, sus_f16, mix_f16, traffic=RAGGED_TRAFFIC_BYTES, traffic_source=TRAFFIC_SOURCE,
                                               kernel="prefill_kernel<F16,128,varlen>", algorithmic_flops=vflops)}
    rec["rope_kv_append_q8_0"] = {"value": a8_gbs, "unit": "GB/s", "ms": a8_avg_ms, "median_ms": a8_med_ms,
                                  "workload": "the rope_kv_append workload into Q8_0 caches, uint8 [8,8,4096,136]",
                                  "roofline": {"bound": "hbm", "achieved": a8_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": a8_gbs / PEAK_HBM_GBS,
                                               "traffic": APPEND_Q8_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE, "kernel": "rope_kernel<F16,neox,fused append,Q8_0>", "algorithmic_bytes": a8bytes}}
    rec["rope"] = {"value": r_gbs, "unit": "GB/s", "ms": r_avg_ms, "median_ms": r_med_ms,
                   "workload": "il_rope in place, x [8,4096,48,128] fp16, rotary_dim 64, base 1e6, start_pos 2048 (reference test/kernels.py:76-96)",
                   "roofline": {"bound": "hbm", "achieved": r_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": r_gbs / PEAK_HBM_GBS,
                                "traffic": ROPE_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE, "kernel": "rope_kernel<F16,interleaved,in place>", "algorithmic_bytes": rbytes}}
    rec["rope_kv_append"] = {"value": a_gbs, "unit": "GB/s", "ms": a_avg_ms, "median_ms": a_med_ms,
                             "workload": "NeoX rope(q) in place + rope(k), v appended to the cache: B=8 L=4096 Hq=32 Hkv=8 D=128 fp16, rotary_dim 128, base 5e5",
                             "roofline": {"bound": "hbm", "achieved": a_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": a_gbs / PEAK_HBM_GBS,
                                          "traffic": APPEND_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE, "kernel": "rope_kernel<F16,neox,fused append>", "algorithmic_bytes": abytes}}
    rec["rope_kv_append_norm"] = {"value": an_gbs, "unit": "GB/s", "ms": an_avg_ms, "median_ms": an_med_ms,
                                  "workload": "the rope_kv_append workload with per-head RMSNorm of q and k (eps 1e-6) applied before the rotation, one launch",
                                  "roofline": {"bound": "hbm", "achieved": an_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": an_gbs / PEAK_HBM_GBS,
                                               "traffic": APPEND_NORM_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE, "kernel": "rope_norm_append_kernel<F16,neox>", "algorithmic_bytes": abytes}}
    rec["qkv"] = {"value": p_tf, "unit": "TFLOP/s", "ms": p_avg_ms, "median_ms": p_med_ms,
                  "workload": "q,k,v = x wq^T, x wk^T, x wv^T in one launch: x [1,4096,4096], wq [4096,4096], wk and wv [1024,4096] fp16 (Llama-3-8B prefill)",
                  "roofline": mfma_roofline(p_tf, sus_f16, traffic=QKV_TRAFFIC_BYTES, traffic_source=TRAFFIC_SOURCE,
                                            kernel="gemm_kernel<F16,[N,K],256x192,grouped,columns numbered through>", algorithmic_flops=pflops)}
    rec["gemm_q8_0"] = {"value": q8_gbs, "unit": "GB/s", "ms": q8_avg_ms, "median_ms": q8_med_ms, "ms_weight_cached": q8_cached_ms,
                        "workload": "one token against a weight of Q8_0 blocks: x [1,1,4096] fp16, W uint8 [14336, 4352] (Llama-3-8B FFN up), out fp16; "
                                    "the calls cycle over 11 copies of the weight (655 MiB), so every call streams it from memory",
                        "roofline": {"bound": "hbm", "achieved": q8_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": q8_gbs / PEAK_HBM_GBS,
                                     "traffic": GEMM_Q8_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE, "kernel": "gemv_q8_kernel<activations in registers>", "algorithmic_bytes": q8bytes}}
    rec["gemm_decode"] = {"value": gd_gbs, "unit": "GB/s", "ms": gd_avg_ms, "median_ms": gd_med_ms, "ms_weight_cached": gd_cached_ms,
                          "workload": "64 decode tokens against an fp16 weight stored [N, K]: x [1,64,4096], W [14336,4096] (Llama-3-8B FFN up), out fp16; weight-streaming, HBM-bound; "
                                      "the calls cycle over 6 copies of the weight (672 MiB), so every call streams it from memory",
                          "roofline": {"bound": "hbm", "achieved": gd_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gd_gbs / PEAK_HBM_GBS,
                                       "traffic": GEMM_DECODE_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE, "kernel": "gemm_stripe_kernel<F16,4>", "algorithmic_bytes": gdbytes}}
    rec["cpu_plumbing"] = {"value": cflops / (c_avg_ms * 1e-3) / 1e12, "unit": "TFLOP/s", "ms": c_avg_ms, "median_ms": c_med_ms,
                           "workload": "prefill B=1 Hq=8 Hkv=2 S=256 D=64 causal dense-mask, fp32 inputs rounded to fp16 for the GPU op (BASELINE configs[0]); launch-bound"}
    rec["calibration"] = {"mfma_only_f16_random": sus_f16, "mfma_only_bf16_random": sus_bf16,
                          "attention_mix_f16_random": mix_f16, "attention_mix_bf16_random": mix_bf16,
                          "note": "mfma_only: v_mfma_f32_16x16x32 alone (the instruction the prefill and GEMM kernels use), two waves per SIMD on every compute unit, operands 0.5*N(0,1); "
                                  "attention_mix: the prefill kernel's per-tile instructions (64 MFMAs, 48 LDS fragment reads, the softmax's vector work) "
                                  "on tiles that stay in LDS, nothing else in the loop; frac_of_sustained and frac_of_attention_mix = achieved / these, "
                                  "reported beside frac (= achieved / nominal peak), measured in this run on this box"}
    rec["rmsnorm"] = {"value": n_gbs, "unit": "GB/s", "ms": n_avg_ms, "median_ms": n_med_ms,
                      "workload": "rmsnorm per token, x [8,4096,6144] fp16, eps 1e-6 (reference test/kernels.py:59-74)",
                      "roofline": {"bound": "hbm", "achieved": n_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": n_gbs / PEAK_HBM_GBS,
                                   "traffic": NORM_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE, "kernel": "rmsnorm_rows_kernel<F16,64,12,streamed>", "algorithmic_bytes": nbytes}}
    rec["gemm"] = {"value": g_tf, "unit": "TFLOP/s", "ms": g_avg_ms, "median_ms": g_med_ms,
                   "workload": "gemm alpha=1 beta=0, A [1,4096,4096] x W [4096,4096] fp16 (reference README HGEMM table, M=K=N=4096)",
                   "published_reference_us": 605.3,
                   "roofline": mfma_roofline(g_tf, sus_f16, traffic=GEMM_TRAFFIC_BYTES, traffic_source=TRAFFIC_SOURCE,
                                             kernel="gemm_kernel<F16,[K,N],256x256>", algorithmic_flops=gflops)}
    mark_stale_traffic(rec)
    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline(torch, workloads, refs, L)
        rec["decode"]["cpu_baseline"] = cpu_baseline_decode(torch, workloads, refs)
        rec["ragged"]["cpu_baseline"] = cpu_baseline_ragged(torch, workloads, refs)
        rec["long_context"]["cpu_baseline"] = cpu_baseline_long(torch, workloads, refs)
        rec["cpu_plumbing"]["cpu_baseline"] = cpu_baseline_plumbing(torch, workloads, refs)
        rec["rope"]["cpu_baseline"] = rope_cpu_baseline(torch, workloads, refs)
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
