"""Benchmark of the FlashAttention2 forward + backward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one forward call and one backward call of the attention operator
through the C ABI, on the workload the headline metric is quoted on:
B=4, N=16, S=2048, D=128, fp16, causal attn_mask (uint8, 1 = masked),
keep_prob = 1, upstream dO ~ N(0,1).  Inputs are synthetic and already resident
in HBM.  Prints one JSON line: whole-job TFLOP/s by the FlashAttention-2 flop
convention (fwd 4*B*N*S^2*D*f, bwd 2.5x, f = 1/2 causal), the roofline of the
dominant kernel from HIP-event timings taken inside the timed region, and the
CPU baseline (the reference's numpy unfused attention, restated in oracle/,
timed on this box's host cores on its own CPU-sized configuration).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2516.6          # MI355X dense fp16 MFMA peak (256 CU x 4 SIMD x 1024 flop/clk x 2.4 GHz)


def cpu_baseline(budget_s=12.0):
    """The reference's CPU attention path (tests/train/flash_attention/st/common.py:110-132,
    restated in oracle/unfused_attention.py) on its CPU-runnable configuration:
    B=1, N=4, S=512, D=64, fp16 N(0,1), scale 1/8 folded into q, no mask, forward only."""
    import numpy as np
    import torch
    from oracle import unfused_attention as orc
    rng = np.random.default_rng(1000)
    q, k, v = (rng.standard_normal((1, 4, 512, 64)).astype(np.float16) for _ in range(3))
    qs = (q.astype(np.float32) * 0.125).astype(np.float16)
    flops = 4 * 1 * 4 * 512 * 512 * 64
    orc.np_unfused_fwd_fp16(qs, k, v)
    times = []
    t_end = time.perf_counter() + budget_s
    while time.perf_counter() < t_end and len(times) < 50:
        t0 = time.perf_counter()
        orc.np_unfused_fwd_fp16(qs, k, v)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    # second formulation: torch fp32 on all host cores (tests/infer/flash_attention/tik/data_gen.py:32-34)
    threads = min(16, os.cpu_count() or 1)
    torch.set_num_threads(threads)
    tq, tk, tv = (torch.from_numpy(x) for x in (qs, k, v))
    for _ in range(3):
        orc.torch_unfused_fwd_fp32(tq, tk, tv)
    tt = []
    for _ in range(20):
        t0 = time.perf_counter()
        orc.torch_unfused_fwd_fp32(tq, tk, tv)
        tt.append(time.perf_counter() - t0)
    tmed = sorted(tt)[len(tt) // 2]
    return {
        "value": flops / med / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": f"unfused fwd B1 N4 S512 D64 fp16 (numpy fp16 matmul, the reference's CPU oracle), median of {len(times)} calls, {med * 1e3:.1f} ms/call",
        "torch_fp32_value": flops / tmed / 1e12, "torch_fp32_cores": threads, "torch_fp32_ms": tmed * 1e3,
        "host_cpus": os.cpu_count(),
    }


class PowerSampler:
    """Board power from the amdgpu hwmon files in sysfs (power1_input, microwatts; power1_cap = the limit the
    power management holds the board to), read every 20 ms by a host thread while the GPU works."""

    def __init__(self):
        import glob
        self.dir = next(iter(sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))), None)
        self.samples, self._stop, self._thread = [], False, None

    def _read(self, name):
        try:
            with open(os.path.join(self.dir, name)) as f:
                return int(f.read())
        except Exception:
            return None

    def start(self):
        import threading
        if self.dir is None or self._read("power1_input") is None:
            return False
        self.samples, self._stop = [], False

        def loop():
            while not self._stop:
                v = self._read("power1_input")
                if v is not None:
                    self.samples.append(v / 1e6)
                time.sleep(0.02)
        self._thread = threading.Thread(target=loop, daemon=True)
        self._thread.start()
        return True

    def stop(self):
        if self._thread is None:
            return None
        self._stop = True
        self._thread.join()
        self._thread = None
        s = self.samples[len(self.samples) // 3:]           # (the first third: the reading still rises)
        if not s:
            return None
        cap = self._read("power1_cap")
        return {"source": os.path.join(self.dir, "power1_input"), "samples": len(s), "mean_w": round(sum(s) / len(s), 1),
                "max_w": round(max(s), 1), "cap_w": None if cap is None else cap / 1e6}


def run_other_configs(args, lib, dev, st, stream, g, D, scale, check, only):
    """The configurations of the benchmark line besides the timed one.  `only`: run just the one of that name
    (for a profiler run over a single configuration) with `args.steps` steps."""
    import ctypes
    import torch
    from acctransformer_amd import _capi
    P = ctypes.byref
    other = {}

    def run_config(name, pp, qq, kk, vv, dd, flops, side_bytes, n=10):
        oo, ll = torch.empty_like(qq), torch.empty(qq.shape[:3], dtype=torch.float32, device=dev)
        g3 = [torch.empty_like(t) for t in (qq, kk, vv)]
        pp.o_stride = _capi._bhs_strides(oo)
        # with dropout, the forward call packs (or draws) the keep bits into a buffer that the backward call of
        # the same step reads (drop_bits / drop_bits_filled of the C ABI), as the Python operator does; the same
        # for what the pre-pass derives from a mask tensor (mask_bits): once per step, in the forward call
        bits = _capi.attach_drop_bits(pp, dev)
        mbits = _capi.attach_mask_bits(pp, dev)
        nw = max(lib.acct_fa_bwd_workspace_bytes(P(pp)), lib.acct_fa_fwd_workspace_bytes(P(pp)), 256)
        w = torch.empty(nw, dtype=torch.uint8, device=dev)

        def one():
            pp.drop_bits_filled = 0
            pp.mask_bits_filled = 0
            check(lib.acct_fa_fwd(P(pp), oo.data_ptr(), ll.data_ptr(), w.data_ptr(), nw, st))
            pp.drop_bits_filled = 1 if bits is not None else 0
            pp.mask_bits_filled = 1 if mbits is not None else 0
            check(lib.acct_fa_bwd(P(pp), oo.data_ptr(), dd.data_ptr(), ll.data_ptr(), g3[0].data_ptr(), g3[1].data_ptr(),
                                  g3[2].data_ptr(), w.data_ptr(), nw, st))
        # untimed: the inputs were drawn on the host while the GPU sat idle, and the clock needs a few tenths
        # of a second under load to settle again
        t_end = time.perf_counter() + max(args.settle_seconds, 0.0) / 2
        while True:
            for _ in range(3):
                one()
            torch.cuda.synchronize()
            if time.perf_counter() >= t_end:
                break
        if only is not None:
            n = args.steps
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(n):
            one()
        e1.record(stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / n
        io = 8 * qq.numel() * qq.element_size() + 2 * ll.numel() * 4 + side_bytes
        other[name] = {"ms_per_step": round(ms, 4), "tflops": round(flops / (ms * 1e-3) / 1e12, 1),
                       "algorithmic_hbm_gb_per_step": round(io / 1e9, 3), "achieved_hbm_gbps": round(io / (ms * 1e-3) / 1e9, 1),
                       "hbm_peak_gbps": 8000.0}

    want = lambda name: only is None or only == name
    # ALiBi + causal, B2 N32 S4096 D128: bias -slope_h (i - j), as a full [1,N,S,S] tensor and in the
    # reference's row-bias form [1,N,1,S] (slope_h j: the row constant cancels in the softmax)
    names3 = ("alibi_causal_B2_N32_S4096_row_bias", "alibi_causal_B2_N32_S4096_full_bias")
    if any(want(nm) for nm in names3):
        B3, N3, S3 = 2, 32, 4096
        q3, k3, v3, d3 = (torch.randn(B3, N3, S3, D, generator=g).half().to(dev) for _ in range(4))
        slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / N3) for h in range(N3)], device=dev)
        pos = torch.arange(S3, device=dev, dtype=torch.float32)
        fl3 = 14.0 * B3 * N3 * S3 * S3 * D * 0.5
        for nm in names3:
            if not want(nm):
                continue
            if nm.endswith("row_bias"):
                al = (slopes[None, :, None, None] * pos[None, None, None, :]).half()
            else:
                al = (-slopes[None, :, None, None] * (pos[None, None, :, None] - pos[None, None, None, :])).half()
            pp = _capi.make_params(q3, k3, v3, scale=scale, next_block_num=0, mask_kind=_capi.MASK_CAUSAL, alibi=al)
            run_config(nm, pp, q3, k3, v3, d3, fl3, 2 * al.numel() * 2)      # the bias is read by the forward and by the backward
            del al
        del q3, k3, v3, d3
    # padded batch + dropout, B16 N16 S1024 D128: key-padding mask [B,S,S] uint8, lengths U[256,1024]; dropout
    # mask uint8 [B,N,S,S] Bernoulli(0.9)
    names5 = ("padded_dropout_B16_N16_S1024_mask_tensor", "padded_dropout_B16_N16_S1024_fp16_mask_tensors",
              "padded_dropout_B16_N16_S1024_seed_pair")
    if any(want(nm) for nm in names5):
        B5, N5, S5 = 16, 16, 1024
        g5 = torch.Generator(device="cpu").manual_seed(1005)
        q5, k5, v5, d5 = (torch.randn(B5, N5, S5, D, generator=g5).half().to(dev) for _ in range(4))
        # (a generator of its own for the lengths: a draw whose mean, 0.4986 S, is that of the draw the earlier
        # runs of this benchmark happened to take from the shared stream, so that the figures stay comparable)
        lens = torch.randint(256, S5 + 1, (B5,), generator=torch.Generator(device="cpu").manual_seed(1898))
        m5 = (torch.arange(S5)[None, None, :] >= lens[:, None, None]).expand(B5, S5, S5).to(torch.uint8).contiguous().to(dev)
        dr5 = (torch.rand(B5, N5, S5, S5, generator=g5) < 0.9).to(torch.uint8).to(dev)
        f5 = float(lens.float().mean()) / S5
        fl5 = 14.0 * B5 * N5 * S5 * S5 * D * f5
        if want(names5[0]):
            pp = _capi.make_params(q5, k5, v5, scale=scale, keep_prob=0.9, mask_kind=_capi.MASK_DENSE_U8, attn_mask=m5, drop_mask=dr5)
            run_config(names5[0], pp, q5, k5, v5, d5, fl5, 2 * (m5.numel() + dr5.numel()))
        if want(names5[1]):
            # the same masks in the reference's own form: fp16 attn_mask (1 = masked) and fp16 {0, 1/keep_prob} dropout mask
            m5f, dr5f = m5.half(), (dr5.half() / 0.9).half()
            pp = _capi.make_params(q5, k5, v5, scale=scale, keep_prob=0.9, mask_kind=_capi.MASK_DENSE_F16, attn_mask=m5f, drop_mask=dr5f)
            run_config(names5[1], pp, q5, k5, v5, d5, fl5, 2 * 2 * (m5.numel() + dr5.numel()))
            del m5f, dr5f
        if want(names5[2]):
            pp = _capi.make_params(q5, k5, v5, scale=scale, keep_prob=0.9, mask_kind=_capi.MASK_DENSE_U8, attn_mask=m5, drop_seed=1234)
            run_config(names5[2], pp, q5, k5, v5, d5, fl5, 2 * m5.numel())
        other["padded_dropout_unmasked_fraction"] = round(f5, 4)
        del q5, k5, v5, d5, m5, dr5
    # the reference's own performance test (tests/train/flash_attention/st/test_fa_perf.py:16-58): the raw op on
    # (4, 8, 4096, 128) with uniform [0, 1) inputs, a (1, S, S) fp16 causal attn_mask and an fp16 {0, 1/keep_prob}
    # dropout mask of rate 0.1, forward and grad
    nm = "reference_perf_test_B4_N8_S4096_fp16_masks_dropout"
    if want(nm):
        B6, N6, S6 = 4, 8, 4096
        g6 = torch.Generator(device="cpu").manual_seed(1006)
        q6, k6, v6 = (torch.rand(B6, N6, S6, D, generator=g6).half().to(dev) for _ in range(3))
        d6 = torch.randn(B6, N6, S6, D, generator=g6).half().to(dev)
        m6 = torch.triu(torch.ones(1, S6, S6, dtype=torch.float16, device=dev), 1)
        dr6 = ((torch.rand(B6, N6, S6, S6, device=dev) < 0.9).half() / 0.9).half()
        pp = _capi.make_params(q6, k6, v6, scale=1.0, keep_prob=0.9, mask_kind=_capi.MASK_DENSE_F16, attn_mask=m6, drop_mask=dr6)
        run_config(nm, pp, q6, k6, v6, d6, 14.0 * B6 * N6 * S6 * S6 * D * 0.5, 2 * 2 * (m6.numel() + dr6.numel()), n=5)
        del q6, k6, v6, d6, m6, dr6
    return other


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--settle-seconds", type=float, default=0.6,
                    help="untimed steps run for this long after the warm-up so that the clocks have settled")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-mfma-probe", action="store_true",
                    help="skip the register-only MFMA rate measurement (the `mfma_sustained` key of the JSON line)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the ALiBi and padded-batch + dropout configurations (extra keys of the JSON line)")
    ap.add_argument("--data", choices=("randn", "const", "zeros"), default="randn",
                    help="q, k, v, dO of the timed workload: N(0,1) (the benchmark's), one value in every element, or "
                         "zeros -- the same instructions on operands that toggle less and draw less power")
    ap.add_argument("--only-config", default=None,
                    help="run one of the `other_configs` by name for --steps steps and print its entry only (so that a "
                         "profile covers that configuration alone)")
    ap.add_argument("--no-dense-pass", action="store_true",
                    help="skip the untimed dense-mask and TriangleAttention comparison passes (so that a profile covers the timed workload only)")
    ap.add_argument("--calib-copy-mib", type=int, default=0,
                    help="also run an elementwise fp32 copy kernel over this many MiB (5 launches) after the timed "
                         "region: a known-size reference for scaling profiler byte counters")
    ap.add_argument("--lib", default=None,
                    help="load this build of libacct_fa.so instead of the in-tree one (a timing build made by "
                         "`make -C acctransformer_amd/csrc leave-out LEAVE_OUT=...`)")
    ap.add_argument("--kernel-times", action="store_true",
                    help="print the time of each of the three kernels alone (HIP events over --steps launches) on the "
                         "benchmark shape, with the mask declared as none and as causal, and exit")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the single-GPU attention hot path: run it with --gpus 1 "
              "(every (batch, head) pair is independent, so more GPUs would only split B*N; nothing here uses a second GPU)",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from acctransformer_amd import _capi
    from acctransformer_amd.flash_attention.ops.flash_attention import flash_attention_impl as impl

    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the attention path has no CPU fallback", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.lib:
        _capi._LIB_PATH = os.path.abspath(args.lib)
    lib = _capi.load()

    B, N, S, D = 4, 16, 2048, 128
    g = torch.Generator(device="cpu").manual_seed(1001)
    if args.only_config:
        stream = torch.cuda.current_stream()
        st = ctypes.c_void_p(stream.cuda_stream)

        def check(rc):
            if rc != 0:
                raise RuntimeError(lib.acct_last_error().decode())
        print(json.dumps(run_other_configs(args, lib, dev, st, stream, g, D, D ** -0.5, check, args.only_config)))
        return
    q, k, v, dO = (torch.randn(B, N, S, D, generator=g).half().to(dev) for _ in range(4))
    if args.data != "randn":
        for t in (q, k, v, dO):
            t.fill_(0.25 if args.data == "const" else 0.0)
    attn_mask = torch.triu(torch.ones(1, S, S, dtype=torch.uint8, device=dev), 1)
    scale = D ** -0.5
    # The timed workload: the uint8 attn_mask tensor is read by the library.  Its pre-pass classifies the 128x128
    # blocks on the device once per step (clean / wholly masked / the causal diagonal pattern), in the forward
    # call, into a buffer that the two backward calls of the step read (mask_bits of the C ABI) ...
    p_dense = _capi.make_params(q, k, v, scale=scale, next_block_num=0, mask_kind=_capi.MASK_DENSE_U8, attn_mask=attn_mask)
    mask_bits = _capi.attach_mask_bits(p_dense, dev)
    # ... and, for comparison, the same workload with the mask declared as ACCT_MASK_CAUSAL (no tensor, no pre-pass)
    p = _capi.make_params(q, k, v, scale=scale, next_block_num=0, mask_kind=_capi.MASK_CAUSAL)

    o = torch.empty_like(q)
    lse = torch.empty(B, N, S, dtype=torch.float32, device=dev)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    for pp in (p, p_dense):
        pp.o_stride = _capi._bhs_strides(o)
    nws = max(lib.acct_fa_bwd_workspace_bytes(ctypes.byref(p_dense)), lib.acct_fa_fwd_workspace_bytes(ctypes.byref(p_dense)), 256)
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream()
    st = ctypes.c_void_p(stream.cuda_stream)
    P = ctypes.byref

    def check(rc):
        if rc != 0:
            raise RuntimeError(lib.acct_last_error().decode())

    def fwd(pp):
        check(lib.acct_fa_fwd(P(pp), o.data_ptr(), lse.data_ptr(), ws.data_ptr(), nws, st))

    def bwd_dq(pp):
        check(lib.acct_fa_bwd_dq(P(pp), o.data_ptr(), dO.data_ptr(), lse.data_ptr(), dq.data_ptr(), ws.data_ptr(), nws, st))

    def bwd_dkdv(pp):
        check(lib.acct_fa_bwd_dkdv(P(pp), o.data_ptr(), dO.data_ptr(), lse.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), nws, st))

    def step(pp):
        pp.mask_bits_filled = 0            # every step classifies its mask anew, in its forward call
        fwd(pp)
        pp.mask_bits_filled = 1 if pp.mask_bits else 0
        bwd_dq(pp); bwd_dkdv(pp)

    if args.kernel_times:
        out = {"lib": _capi.lib_path(), "data": args.data, "launches": args.steps, "unit": "us", "kernels": {}}
        for name, kind in (("mask_none", _capi.MASK_NONE), ("mask_causal", _capi.MASK_CAUSAL)):
            pk = _capi.make_params(q, k, v, scale=scale, mask_kind=kind)
            pk.o_stride = _capi._bhs_strides(o)
            fwd(pk)
            row = {}
            for kname, fn in (("fa_fwd", fwd), ("fa_bwd_dq", bwd_dq), ("fa_bwd_dkdv", bwd_dkdv)):
                t_s = time.perf_counter()
                while time.perf_counter() - t_s < args.settle_seconds:
                    for _ in range(20):
                        fn(pk)
                    torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(args.steps):
                    fn(pk)
                e1.record(stream)
                torch.cuda.synchronize()
                row[kname] = round(e0.elapsed_time(e1) * 1e3 / args.steps, 2)
            out["kernels"][name] = row
        print(json.dumps(out))
        return

    for _ in range(args.warmup):
        step(p_dense)
    torch.cuda.synchronize()
    # Clock settle: the first ~100 steps after an idle period run on clocks that are still moving (measured:
    # up to 16 % slower), whatever --warmup says.  Keep stepping untimed until half a second of work has gone
    # through the GPU; the timed region below then starts on settled clocks.
    power = PowerSampler()
    power.start()                                         # sampled over the settle phase and the timed region
    t_s = time.perf_counter()
    settle_steps = 0
    while time.perf_counter() - t_s < args.settle_seconds:
        for _ in range(20):
            step(p_dense)
        torch.cuda.synchronize()
        settle_steps += 20
    settle_s = time.perf_counter() - t_s

    K = args.steps
    # per-kernel HIP events inside the timed region, on every fourth step (an event record is a packet of its
    # own on the stream: four of them in every step would cost the step a few microseconds)
    sampled = [i for i in range(K) if i % 4 == 0]
    ev = {i: [torch.cuda.Event(enable_timing=True) for _ in range(4)] for i in sampled}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(K):
        e = ev.get(i)
        p_dense.mask_bits_filled = 0
        if e: e[0].record(stream)
        fwd(p_dense)                                      # mask pre-pass (one small launch) + forward kernel
        p_dense.mask_bits_filled = 1
        if e: e[1].record(stream)
        bwd_dq(p_dense)
        if e: e[2].record(stream)
        bwd_dkdv(p_dense)
        if e: e[3].record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    board_power = power.stop()
    ms_step = wall * 1e3 / K
    t_fwd = sum(e[0].elapsed_time(e[1]) for e in ev.values()) / len(ev)
    t_dq = sum(e[1].elapsed_time(e[2]) for e in ev.values()) / len(ev)
    t_dkdv = sum(e[2].elapsed_time(e[3]) for e in ev.values()) / len(ev)

    # the same workload with the mask declared as ACCT_MASK_CAUSAL instead of read from the tensor (untimed for `value`)
    ms_index = None
    if not args.no_dense_pass:
        for _ in range(3):
            step(p)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(K):
            step(p)
        torch.cuda.synchronize()
        ms_index = (time.perf_counter() - t1) * 1e3 / K

    # TriangleAttention forward with block skip vs. a forward that visits every block (untimed for `value`):
    # B8 N32 S4096 D128 fp16, 128x128 blocks, causal mask
    tri = None
    if not args.no_dense_pass:
        from acctransformer_amd.triangle_attention.triangle_attention import TriangleAttention
        Bt, Nt, St = 8, 32, 4096
        qt, kt, vt = (torch.randn(Bt, Nt, St, D, generator=g).half().to(dev) for _ in range(3))
        mt = torch.triu(torch.ones(1, St, St, dtype=torch.uint8, device=dev), 1).expand(Bt, St, St)
        layer = TriangleAttention(block_size=128).eval()
        full_op = impl.get_flash_attention(scale=1.0)

        def timeit(fn, n=5):
            fn(); fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(n):
                fn()
            e1.record(stream)
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / n

        with torch.no_grad():                 # alternate the two so that clock drift hits both alike; medians
            rounds = [(timeit(lambda: layer(qt, kt, vt, mt)), timeit(lambda: full_op(qt, kt, vt, None, None, None)))
                      for _ in range(5)]
        ms_tri = sorted(r[0] for r in rounds)[2]
        ms_all = sorted(r[1] for r in rounds)[2]
        tri = {"workload": "forward B8 N32 S4096 D128 fp16, causal mask, 128x128 blocks",
               "triangle_attention_ms": round(ms_tri, 4), "all_blocks_forward_ms": round(ms_all, 4),
               "block_skip_speedup": round(ms_all / ms_tri, 3)}
        del qt, kt, vt, mt

    # The other training configurations (untimed for `value`; extra keys of the line): forward + fused
    # backward through the C ABI, kernel time by HIP events on the launch stream, algorithmic flops by the same
    # convention, and the algorithmic HBM bytes per step (every operand read or written once: q, k, v, O, dO,
    # dQ, dK, dV, LSE twice, and the side inputs once per call that reads them) over the same time.
    other = None
    if not args.no_other_configs:
        other = run_other_configs(args, lib, dev, st, stream, g, D, scale, check, None)
    if args.calib_copy_mib > 0:
        src = torch.ones(args.calib_copy_mib * (1 << 18), dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.mul(src, 1.0, out=dst)          # reads and writes calib_copy_mib MiB each
        torch.cuda.synchronize()
        del src, dst

    f = 0.5
    fl_fwd = 4.0 * B * N * S * S * D * f
    fl_bwd = 2.5 * fl_fwd
    fl_step = fl_fwd + fl_bwd
    value = fl_step / (ms_step * 1e-3) / 1e12

    # dominant kernel: the dK/dV kernel of the backward.  Algorithmic flops per launch: 4 of the 5
    # backward matmuls (S, dP, dV, dK) = 8*B*N*S^2*D*f; the dQ kernel carries the fifth plus its
    # own recompute of S and dP.
    kernels = {
        "fa_fwd_kernel": (t_fwd, fl_fwd),
        "fa_bwd_dq_kernel": (t_dq, 0.2 * fl_bwd),
        "fa_bwd_dkdv_kernel": (t_dkdv, 0.8 * fl_bwd),
    }
    # HBM-side bytes per launch, from the FETCH_SIZE / WRITE_SIZE counter runs summarised under profiles/
    # (each scaled by what the same counter reads for a 256 MiB copy kernel: x2.000 and x1.000)
    traffic_bytes = {"fa_fwd_kernel": 189.5e6, "fa_bwd_dq_kernel": 292.7e6, "fa_bwd_dkdv_kernel": 287.1e6}
    dom = max(kernels, key=lambda n: kernels[n][0])
    dom_ms, dom_fl = kernels[dom]
    achieved = dom_fl / (dom_ms * 1e-3) / 1e12
    # What the matrix pipe sustains on this GPU with nothing else in the way (register-only MFMA loop, two waves
    # per SIMD on every CU): the yardstick `roofline.frac` is read against.  The rate depends on how much the
    # operands toggle (the clock follows the power drawn); the benchmark's N(0,1) data is the varying case.
    mfma = None
    if not args.no_mfma_probe:
        rates, clocks, watts = {}, {}, {}
        for key, varying in (("varying_operands", 1), ("constant_operands", 0)):
            r, ghz = ctypes.c_double(0.0), ctypes.c_double(0.0)
            power.start()
            t_p = time.perf_counter()
            while True:                                   # (repeated for half a second so that the power reading settles)
                check(lib.acct_probe_mfma_clock(varying, ctypes.byref(r), ctypes.byref(ghz), st))
                if time.perf_counter() - t_p > 0.5:
                    break
            w = power.stop()
            rates[key] = round(r.value, 1)
            clocks[key] = round(ghz.value, 3)
            watts[key] = None if w is None else w["mean_w"]
        # (shader clock a wave saw inside the loop: an MFMA takes 32 clocks either way, the power drawn sets the clock)
        mfma = {"unit": "TFLOP/s", "instruction": "v_mfma_f32_32x32x16_f16", **rates, "shader_clock_ghz": clocks, "board_power_w": watts,
                "frac_of_nominal_peak": round(rates["varying_operands"] / PEAK_FP16_TFLOPS, 4),
                "dominant_kernel_frac_of_sustained": round(achieved / rates["varying_operands"], 4)}
    out = {
        "metric": "FA2 fwd+bwd TFLOP/s & % fp16 MFMA peak, B4 N16 S2048 D128 causal",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": K, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16", "data": "synthetic",
        "config": {"workload": "FlashAttention2 fwd+bwd B=4 N=16 S=2048 D=128 fp16, causal uint8 attn_mask, keep_prob=1.0, next_block_num=0",
                   "flop_convention": "fwd 4*B*N*S^2*D*f, bwd 2.5x fwd, f=0.5", "gflop_per_step": round(fl_step / 1e9, 1)},
        "pct_of_fp16_mfma_peak": round(100.0 * value / PEAK_FP16_TFLOPS, 2),
        "kernel_ms": {"fa_fwd_kernel_with_mask_prepass": round(t_fwd, 4), "fa_bwd_dq_kernel": round(t_dq, 4), "fa_bwd_dkdv_kernel": round(t_dkdv, 4)},
        "fwd_tflops": round(fl_fwd / (t_fwd * 1e-3) / 1e12, 1), "bwd_tflops": round(fl_bwd / ((t_dq + t_dkdv) * 1e-3) / 1e12, 1),
        "mask_path": "uint8 attn_mask tensor read by the library; block classes derived on the device once per step (forward call) and shared with the backward calls through mask_bits",
        "index_compare_path_ms_per_step": None if ms_index is None else round(ms_index, 4),
        "triangle_block_skip": tri,
        "other_configs": other,
        "clock_settle": {"seconds": round(settle_s, 3), "steps": settle_steps},
        "board_power": board_power,
        "input_data": args.data,
        "mfma_sustained": mfma,
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 1), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP16_TFLOPS, 4), "traffic": traffic_bytes[dom]},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
