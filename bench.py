#!/usr/bin/env python3
"""Float8Linear fwd+bwd throughput at LLaMa-2-70B linear shapes on one MI355X.

One "step" = forward + backward (dynamic scaling on input, weight and grad_output)
through each of the four 70B linear shapes at M = 16384 tokens, inputs resident in
HBM.  Prints ONE JSON line: whole-job TFLOP/s (3 * 2*M*K*N flop per shape, the
reference benchmark's convention), the fp8 GEMM kernel's roofline position measured
with HIP events around every launch inside the timed region, the amax / cast
kernels' HBM figures, bf16 nn.Linear on the same GPU, and the CPU oracle timed on
a bounded sample on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

SHAPES = [  # (name, K, N) at M tokens
    ("wqkv", 8192, 10240),
    ("wo", 8192, 8192),
    ("w13", 8192, 57344),
    ("w2", 28672, 8192),
]
M_TOKENS = 16384
PEAK_FP8_TFLOPS = 5000.0  # MI355X dense fp8 MFMA
PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
# Bytes per GEMM launch that cross the L2 boundary (fetch + write), averaged over the 12 launches of a step, come
# from a tracked record of the last rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script (each counter scaled
# by its reading for a 1 GiB device copy), which also names the commit and the workload it was measured at.
GEMM_TRAFFIC_RECORD = os.path.join(ROOT, "profiles", "bench_llama70b_gemm_hbm_traffic.json")


def gemm_traffic(m, scaling):
    """(bytes per GEMM launch past the L2, provenance string) from the tracked profile record; (None, why) when the
    record is missing or was measured on another workload than this run's."""
    try:
        with open(GEMM_TRAFFIC_RECORD) as f:
            rec = json.load(f)
    except (OSError, ValueError) as e:
        return None, f"no record ({type(e).__name__})"
    if rec.get("m_tokens") != m or rec.get("scaling") != scaling:
        return None, f"record is for M={rec.get('m_tokens')}, {rec.get('scaling')} scaling"
    total = rec["fetch_bytes_per_launch"] + rec["write_bytes_per_launch"]
    why = (f"bytes past the L2 per launch: FETCH_SIZE {rec['fetch_bytes_per_launch']:.4g} + WRITE_SIZE "
           f"{rec['write_bytes_per_launch']:.4g} (rocprofv3 --pmc, calibrated on a 1 GiB copy), measured at commit "
           f"{rec.get('commit', '?')} ({os.path.basename(GEMM_TRAFFIC_RECORD)}); algorithmic: "
           f"{rec.get('algorithmic_bytes_per_launch', 1.035e9):.4g}")
    return total, why


def _cuda0_pci_bus_id():
    """PCI address of torch's cuda:0 ("0000:c1:00.0"), or None when torch is not loaded / has no GPU."""
    torch = sys.modules.get("torch")
    try:
        if torch is None or not torch.cuda.is_available():
            return None
        p = torch.cuda.get_device_properties(0)
        return "%04x:%02x:%02x.0" % (p.pci_domain_id, p.pci_bus_id, p.pci_device_id)
    except Exception:
        return None


class Telemetry:
    """Socket power and shader clock of the GPU while the timed region runs, sampled from sysfs by a host thread
    (reads of two small files every 5 ms; nothing on the launch path)."""

    def __init__(self, period=0.005, pci_bus_id=None):
        """``pci_bus_id`` ("0000:c1:00.0"): the card to sample; default: the PCI address of torch's cuda:0 when torch is
        loaded and a GPU is there, else the first card with power telemetry."""
        import glob
        import threading

        if pci_bus_id is None:
            pci_bus_id = _cuda0_pci_bus_id()
        self.period = period
        self.power_w, self.sclk_mhz = [], []
        self.cap_w = None
        self._stop = threading.Event()
        self._thread = None
        self.power_file = self.sclk_file = self.card = None
        cards = sorted(glob.glob("/sys/class/drm/card[0-9]*/device"))
        if pci_bus_id:  # the sysfs entry is a link to the PCI device: .../0000:c1:00.0
            mine = [d for d in cards if os.path.basename(os.path.realpath(d)).lower() == pci_bus_id.lower()]
            cards = mine or cards
        for dev in cards:
            hw = sorted(glob.glob(os.path.join(dev, "hwmon", "hwmon*", "power1_input"))
                        + glob.glob(os.path.join(dev, "hwmon", "hwmon*", "power1_average")))
            if hw and os.path.exists(os.path.join(dev, "pp_dpm_sclk")):
                self.power_file, self.sclk_file = hw[0], os.path.join(dev, "pp_dpm_sclk")
                self.card = os.path.basename(os.path.realpath(dev))
                try:
                    self.cap_w = int(open(os.path.join(os.path.dirname(hw[0]), "power1_cap")).read()) / 1e6
                except (OSError, ValueError):
                    pass
                break

    def _sample(self):
        try:
            self.power_w.append(int(open(self.power_file).read()) / 1e6)
            for line in open(self.sclk_file).read().splitlines():
                if line.rstrip().endswith("*"):  # the current level, e.g. "S: 1795Mhz *"
                    self.sclk_mhz.append(float(line.split(":")[1].strip().split("M")[0]))
        except (OSError, ValueError, IndexError):
            pass

    def _run(self):
        while not self._stop.is_set():
            self._sample()
            self._stop.wait(self.period)

    def start(self):
        import threading

        if self.power_file is None:
            return
        self._thread = threading.Thread(target=self._run, daemon=True)
        self._thread.start()

    def stop(self):
        self._stop.set()
        if self._thread is not None:
            self._thread.join()
        if not self.power_w:
            return None
        mean = lambda v: sum(v) / len(v) if v else None
        return {"source": "sysfs hwmon power1_input + pp_dpm_sclk, every %d ms over the timed region" % int(self.period * 1e3),
                "card": self.card,
                "samples": len(self.power_w), "socket_power_W_mean": mean(self.power_w), "socket_power_W_max": max(self.power_w),
                "power_cap_W": self.cap_w, "sclk_MHz_mean": mean(self.sclk_mhz),
                "sclk_MHz_min": min(self.sclk_mhz) if self.sclk_mhz else None,
                "sclk_MHz_max": max(self.sclk_mhz) if self.sclk_mhz else None}


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=5)
    p.add_argument("--warmup", type=int, default=2)
    p.add_argument("--m", type=int, default=M_TOKENS, help="tokens per step (default: the benchmark's 16384)")
    p.add_argument("--scaling", choices=["dynamic", "delayed"], default="dynamic",
                   help="dynamic (the headline configuration) or delayed scaling of all three tensors with one "
                        "sync_float8_amax_and_scale_history per step")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-bf16", action="store_true")
    p.add_argument("--cpu-seconds", type=float, default=15.0, help="target CPU time of the oracle sample")
    p.add_argument("--mfma-order", type=int, default=0, choices=[0, 1, 2, 3],
                   help="register-only MFMA loop: which operand changes between consecutive instructions "
                        "(0 the first, as in the GEMM; 1 the second; 2 both; 3 neither for eight in a row)")
    p.add_argument("--per-gemm-only", type=float, default=None, metavar="SECONDS",
                   help="run nothing but the twelve products of a step, each alone, through this library and through "
                        "torch._scaled_mm (for profiler runs that compare the two kernels product by product); SECONDS > 0 "
                        "also loops each for that long and samples socket power and shader clock")
    p.add_argument("--no-other-configs", action="store_true",
                   help="leave out the configurations besides the headline one (profiler runs of the headline's kernels)")
    p.add_argument("--calibrate-copy", action="store_true",
                   help="also run one plain 1 GiB device-to-device copy (for scaling hardware byte counters of a profiler run)")
    return p.parse_args()


def make_layers(torch, f8, m, device, scaling="dynamic"):
    layers = []
    if scaling == "delayed":
        cc = f8.CastConfig(f8.ScalingType.DELAYED)
        config = f8.Float8LinearConfig(cast_config_input=cc, cast_config_weight=cc, cast_config_grad_output=cc)
    else:
        config = f8.Float8LinearConfig()
    for name, k, n in SHAPES:
        lin = torch.nn.Linear(k, n, bias=False, device=device, dtype=torch.bfloat16)  # kaiming-uniform init
        mod = f8.Float8Linear.from_float(lin, config=config)
        x = torch.randn(m, k, device=device, dtype=torch.bfloat16).requires_grad_()
        dy = (torch.randn(m, n, device=device, dtype=torch.float32) * 1e-2).to(torch.bfloat16)
        layers.append((name, k, n, lin, mod, x, dy))
    return layers


def step(layers, use_fp8=True, sync=None):
    if sync is not None and use_fp8:
        sync()
    for name, k, n, lin, mod, x, dy in layers:
        x.grad = None
        lin.weight.grad = None
        y = (mod if use_fp8 else lin)(x)
        y.backward(dy)


def timed(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def probe_mfma(torch, random_data, iters=4000, operands=None, seconds=0.8, order=0, idle_w=None):
    """Register-only fp8 MFMA loop on every CU: what the matrix cores sustain with no memory traffic, on zero operands
    (clock limit), random ones (the chip's power / current limits) or -- ``operands``: an fp8 tensor of at least
    256 KiB -- the bytes of a real tensor.  ``order``: which operand changes from one instruction to the next (0 the
    first, as in the GEMM; 1 the second; 2 both; 3 neither for eight in a row).  The loop runs for ``seconds`` and the rate of the last third is reported,
    with the socket power and shader clock over that third: the power management takes some hundred milliseconds to
    settle, and a single 2 ms launch right after the GEMMs reads the clock they left, not the loop's own.
    From libf8mi_probe.so, a bench-only helper next to the library."""
    import ctypes as C

    path = os.path.join(ROOT, "float8_experimental_amd", "libf8mi_probe.so")
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path)
    lib.f8mi_probe_mfma.restype = C.c_int
    lib.f8mi_probe_mfma.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.POINTER(C.c_double), C.c_void_p]
    scratch = torch.empty(1 << 20, dtype=torch.uint8, device="cuda:0")
    mode = int(random_data)
    if operands is not None:
        scratch[:1 << 18].copy_(operands.reshape(-1).view(torch.uint8)[:1 << 18])
        mode = 2
    out = C.c_double(0.0)
    stream = torch.cuda.current_stream().cuda_stream

    def once():
        rc = lib.f8mi_probe_mfma(mode + 16 * order, iters, scratch.data_ptr(), scratch.numel(), C.byref(out), stream)
        return out.value if rc == 0 else None

    t_end = time.perf_counter() + seconds * 2.0 / 3.0
    while time.perf_counter() < t_end:
        if once() is None:
            return None
    tele = Telemetry()
    tele.start()
    vals = []
    t_end = time.perf_counter() + seconds / 3.0
    while time.perf_counter() < t_end:
        vals.append(once())
    t = tele.stop() or {}
    if not vals or any(v is None for v in vals):  # a failed probe call: no figure rather than a wrong one
        return None
    out = {"TFLOP/s": sum(vals) / len(vals), "socket_power_W": t.get("socket_power_W_mean"), "sclk_MHz": t.get("sclk_MHz_mean")}
    if idle_w and out["socket_power_W"]:
        out["pJ_per_flop_above_idle"] = (out["socket_power_W"] - idle_w) / out["TFLOP/s"]
    return out


def vendor_scaled_mm(torch, _native, layers, m, flop_step, iters, seconds=0.0):
    """The same twelve products through torch._scaled_mm (hipBLASLt) on row-major fp8 operands with the transposed
    copies it needs made beforehand -- a reference point for the GEMM kernel, outside the timed region: all twelve back
    to back, and each product alone against this library's kernel on the same bytes (one fp8 copy per tensor, read as
    it lies or transposed).  ``seconds`` > 0: each product is also looped for that long per kernel with the socket
    power and shader clock sampled over the second half (what rate, power and clock each settles at).  An "error" entry
    where the installed torch refuses a product (format pair or layout)."""
    E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2
    bf16 = torch.bfloat16
    rowmajor = lambda t: t.permute(1, 0, 2).reshape(t.shape[1], -1).contiguous()
    transposed = lambda t: t.view(torch.uint8).t().contiguous().view(t.dtype)

    def timed_loop(fn, n):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    def settled(fn, flop):
        t_end = time.perf_counter() + seconds / 2
        while time.perf_counter() < t_end:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
        tele = Telemetry()
        tele.start()
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < seconds / 2:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
            n += 10
        dt = (time.perf_counter() - t0) / n
        t = tele.stop() or {}
        return {"TFLOP/s": flop / dt / 1e12, "socket_power_W": t.get("socket_power_W_mean"), "sclk_MHz": t.get("sclk_MHz_mean")}

    try:
        per_gemm, vendor_all, ours_all = [], [], []
        for name, k, n, lin, mod, x, dy in layers:
            x8, _, sx = _native.cast_dynamic(x.detach(), E4, out_kblock=True)
            w8, _, sw = _native.cast_dynamic(lin.weight.detach(), E4, out_kblock=True)
            g8, _, sg = _native.cast_dynamic(dy, E5, out_kblock=True)
            x8r, w8r, g8r = rowmajor(x8), rowmajor(w8), rowmajor(g8)
            w8t, g8t, x8t = transposed(w8r), transposed(g8r), transposed(x8r)
            # torch._scaled_mm(a, b): a row-major [rows, inner], b column-major [inner, cols] = .t() of a row-major [cols, inner]
            products = (
                ("forward", lambda: _native.gemm_nt_kb(x8, sx, w8, sw, bf16),
                 lambda: torch._scaled_mm(x8r, w8r.t(), scale_a=sx, scale_b=sw, out_dtype=bf16)),
                ("grad_input", lambda: _native.gemm_kb_ex(g8, False, sg, w8, True, sw, bf16),
                 lambda: torch._scaled_mm(g8r, w8t.t(), scale_a=sg, scale_b=sw, out_dtype=bf16)),
                ("grad_weight", lambda: _native.gemm_kb_ex(g8, True, sg, x8, True, sx, bf16),
                 lambda: torch._scaled_mm(g8t, x8t.t(), scale_a=sg, scale_b=sx, out_dtype=bf16)),
            )
            flop = 2.0 * m * k * n
            for what, ours, theirs in products:
                t_ours, t_theirs = timed_loop(ours, iters), timed_loop(theirs, iters)
                row = {"shape": name, "product": what, "this_library_TFLOP/s": flop / t_ours / 1e12,
                       "scaled_mm_TFLOP/s": flop / t_theirs / 1e12}
                if seconds > 0:
                    row["this_library_settled"] = settled(ours, flop)
                    row["scaled_mm_settled"] = settled(theirs, flop)
                per_gemm.append(row)
                vendor_all.append(t_theirs)
                ours_all.append(t_ours)
            del x8, w8, g8, x8r, w8r, g8r, w8t, g8t, x8t, products
        ours_ms = sum(ours_all) * 1e3
        return {"what": "torch._scaled_mm (hipBLASLt), bf16 output; each product alone, back to back with itself",
                "scaled_mm_TFLOP/s": flop_step / sum(vendor_all) / 1e12, "scaled_mm_ms_per_12_gemms": sum(vendor_all) * 1e3,
                "this_library_TFLOP/s": flop_step / (ours_ms * 1e-3) / 1e12, "this_library_ms_per_12_gemms": ours_ms,
                "per_gemm": per_gemm}
    except Exception as e:  # a product this torch build does not take
        return {"scaled_mm_TFLOP/s": None, "error": f"{type(e).__name__}: {str(e)[:160]}"}


def _prof_window(torch, _native, fn, reps):
    """Runs fn() reps times with the library's per-kernel HIP-event counters on; {kernel: (launches, ms, work)}."""
    _native.prof_reset()
    _native.prof_enable(True)
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    _native.prof_enable(False)
    prof = {name: _native.prof_read(kid) for name, kid in (("amax", _native.K_AMAX), ("cast", _native.K_CAST),
                                                           ("gemm", _native.K_GEMM), ("sync", _native.K_SYNC))}
    _native.prof_reset()
    return prof


def _rates(prof, flop=None, reps=1):
    """GEMM TFLOP/s (over ``flop`` algorithmic flop per repetition when given: padded products count their unpadded
    work), cast / amax GB/s and fractions of the peaks, from a _prof_window record."""
    out = {}
    n, ms, work = prof["gemm"]
    if ms > 0:
        f = flop * reps if flop else work
        out["gemm_TFLOP/s"] = f / ms / 1e9
        out["gemm_frac_of_fp8_peak"] = f / ms / 1e9 / PEAK_FP8_TFLOPS
        out["gemm_ms"] = ms / reps
    for k in ("cast", "amax"):
        n, ms, work = prof[k]
        if ms > 0:
            out[f"{k}_GB/s"] = work / ms / 1e6
            out[f"{k}_frac_of_hbm_peak"] = work / ms / 1e6 / PEAK_HBM_GBS
            out[f"{k}_ms"] = ms / reps
    return out


LLAMA3_8B_LINEARS = [  # (name, K, N) of the seven linears of one Llama-3-8B decoder layer (d 4096, ffn 14336, 8 KV heads)
    ("wq", 4096, 4096), ("wk", 4096, 1024), ("wv", 4096, 1024), ("wo", 4096, 4096),
    ("w1", 4096, 14336), ("w3", 4096, 14336), ("w2", 14336, 4096),
]
RAGGED_LAYERS = [(4099, 4097, 11007), (4099, 1000, 3000)]  # (tokens, K, N): no dimension a multiple of 16


def other_configs(torch, f8, _native, layers, args):
    """The benchmark configurations besides the headline one, each outside the headline's timed region and measured
    the same way (wall clock over whole steps, kernel times from HIP events on the launch stream): delayed scaling of
    all three tensors on the same four shapes with one sync per step, the sync kernel's latency at 12 and 240
    (layer, tensor) entries, the seven linear shapes of a Llama-3-8B layer at 8192 tokens, and two ragged layers."""
    dev = torch.device("cuda:0")
    steps = max(2, args.steps)
    out = {}
    DEL = f8.CastConfig(f8.ScalingType.DELAYED)
    delayed_cfg = f8.Float8LinearConfig(cast_config_input=DEL, cast_config_weight=DEL, cast_config_grad_output=DEL)

    def fwd_bwd(mod, x, dy):
        x.grad = None
        mod.weight.grad = None
        mod(x).backward(dy)

    # ---- delayed scaling x3 on the headline's shapes (same weights, inputs and gradients), history 16, one sync per step
    if args.scaling == "dynamic":
        mods = [f8.Float8Linear.from_float(lay[3], config=delayed_cfg) for lay in layers]
        model = torch.nn.ModuleList(mods)

        def dstep():
            f8.sync_float8_amax_and_scale_history(model)
            for mod, lay in zip(mods, layers):
                fwd_bwd(mod, lay[5], lay[6])

        flop = sum(3 * 2.0 * lay[5].shape[0] * lay[1] * lay[2] for lay in layers)
        sec = timed(torch, dstep, steps, 2)
        prof = _prof_window(torch, _native, dstep, 2)
        r = {"ms_per_step": sec * 1e3, "TFLOP/s": flop / sec / 1e12, "history_len": 16,
             "what": "delayed scaling of input, weight and grad_output; sync_float8_amax_and_scale_history over the four "
                     "layers, then fwd+bwd of each; the cast is the fused amax + cast (4 bytes moved per bf16 element incl. "
                     "its finalize launch)"}
        r.update(_rates(prof, reps=2))
        n, ms, _ = prof["sync"]
        r["sync_us_per_launch"] = ms / max(n, 1) * 1e3
        r["sync_entries"] = 3 * len(mods)
        out["delayed_llama70b"] = r
        del mods, model

    # ---- sync latency by number of (layer, tensor) entries: kernel time from HIP events, and the host's wall time per call
    lat = {}
    for n_layers in (4, 80):
        small = torch.nn.ModuleList([f8.Float8Linear.from_float(torch.nn.Linear(64, 64, bias=False, device=dev, dtype=torch.bfloat16),
                                                                config=delayed_cfg) for _ in range(n_layers)])
        for mod in small:
            mod.last_seen_input_dtype = torch.bfloat16
        call = lambda: f8.sync_float8_amax_and_scale_history(small)
        wall = timed(torch, call, 200, 20)
        prof = _prof_window(torch, _native, call, 50)
        n, ms, nbytes = prof["sync"]
        lat[f"{3 * n_layers}_entries"] = {"kernel_us": ms / max(n, 1) * 1e3, "launches_per_call": n / 50,
                                         "host_wall_us_per_call_back_to_back": wall * 1e6, "bytes": nbytes / max(n, 1)}
        del small
    out["sync_latency"] = lat

    # ---- the seven linear shapes of a Llama-3-8B layer at 8192 tokens (dynamic scaling), fwd+bwd each
    tokens = 8192
    per, tot_flop, tot_sec, tot_prof = {}, 0.0, 0.0, None
    for name, k, n in LLAMA3_8B_LINEARS:
        lin = torch.nn.Linear(k, n, bias=False, device=dev, dtype=torch.bfloat16)
        mod = f8.Float8Linear.from_float(lin)
        x = torch.randn(tokens, k, device=dev, dtype=torch.bfloat16).requires_grad_()
        dy = (torch.randn(tokens, n, device=dev) * 1e-2).to(torch.bfloat16)
        flop = 3 * 2.0 * tokens * k * n
        sec = timed(torch, lambda: fwd_bwd(mod, x, dy), 4 * steps, 3)
        prof = _prof_window(torch, _native, lambda: fwd_bwd(mod, x, dy), 4)
        per[name] = {"K": k, "N": n, "ms": sec * 1e3, "TFLOP/s": flop / sec / 1e12, **_rates(prof, flop, 4)}
        tot_flop += flop
        tot_sec += sec
        tot_prof = prof if tot_prof is None else {kk: tuple(a + b for a, b in zip(tot_prof[kk], prof[kk])) for kk in prof}
        del lin, mod, x, dy
    out["llama3_8b_linear_shapes"] = {"tokens": tokens, "ms_all_seven": tot_sec * 1e3, "TFLOP/s": tot_flop / tot_sec / 1e12,
                                      **_rates(tot_prof, tot_flop, 4), "per_shape": per}

    # ---- ragged layers (no dimension a multiple of 16): zero-padded k-blocked fp8 copies, fwd+bwd, against bf16
    rag = {}
    for tokens, k, n in RAGGED_LAYERS:
        lin = torch.nn.Linear(k, n, bias=False, device=dev, dtype=torch.bfloat16)
        mod = f8.Float8Linear.from_float(lin)
        x = torch.randn(tokens, k, device=dev, dtype=torch.bfloat16).requires_grad_()
        dy = (torch.randn(tokens, n, device=dev) * 1e-2).to(torch.bfloat16)
        flop = 3 * 2.0 * tokens * k * n
        sec = timed(torch, lambda: fwd_bwd(mod, x, dy), 10 * steps, 5)
        prof = _prof_window(torch, _native, lambda: fwd_bwd(mod, x, dy), 10)
        r = {"ms": sec * 1e3, "TFLOP/s": flop / sec / 1e12, **_rates(prof, flop, 10),
             # a layer this small is bound by the host in eager mode (about 12 launches per fwd+bwd): the kernels' own time
             "kernel_ms_sum": sum(prof[kk][1] for kk in ("amax", "cast", "gemm")) / 10,
             "kernels": {p: list(_native.linear_route(tokens, k, n)[p][2]) for p in ("output", "grad_input", "grad_weight")}}
        if not args.no_bf16:
            secb = timed(torch, lambda: fwd_bwd(lin, x, dy), 10 * steps, 5)
            r["bf16_ms"] = secb * 1e3
            r["speedup_vs_bf16"] = secb / sec
        rag[f"{tokens}x{k}->{n}"] = r
        del lin, mod, x, dy
    out["ragged_layers"] = rag
    return out


def cpu_baseline(torch, target_s):
    """The oracle's emulate=True restatement (fp32 dequant + torch.mm on the host) on token slices of the benchmark
    shapes, smallest weight first, until about ``target_s`` seconds of CPU work have been timed."""
    from oracle import torch_oracle as to

    torch.manual_seed(0)

    def run(m, k, n, w):
        x = torch.randn(m, k).to(torch.bfloat16)
        dy = (torch.randn(m, n) * 1e-2).to(torch.bfloat16)
        t0 = time.perf_counter()
        to.linear_fwd_bwd_dynamic(x, w, dy)
        return time.perf_counter() - t0

    parts, flop, secs = [], 0.0, 0.0
    for name, k, n in sorted(SHAPES, key=lambda s: s[1] * s[2]):  # wo (8192 x 8192), wqkv (8192 x 10240), w2, w13
        if secs >= 0.7 * target_s:
            break
        w = (torch.rand(n, k) * 2 - 1).mul_(k**-0.5).to(torch.bfloat16)
        if not parts:
            run(256, k, n, w)  # warm the BLAS threads
        t_small = run(512, k, n, w)
        m = 512
        while m < M_TOKENS and secs + t_small * (2 * m / 512) <= target_s:
            m *= 2
        t = run(m, k, n, w)
        parts.append(f"M={m} of {M_TOKENS} tokens of {name} (K={k}, N={n}): {t:.2f} s")
        flop += 3 * 2.0 * m * k * n
        secs += t
        del w
    return {
        "value": flop / secs / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "oracle.torch_oracle.linear_fwd_bwd_dynamic (amax+scale, saturated casts, 3 emulated fp32 GEMMs), one run each on "
                  + "; ".join(parts),
        "seconds": secs,
    }


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build drives ONE GPU (no collectives in the path); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    import float8_experimental_amd as f8
    from float8_experimental_amd import _native

    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    _native.lib()
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    m = args.m
    layers = make_layers(torch, f8, m, dev, args.scaling)
    sync = None
    if args.scaling == "delayed":
        model = torch.nn.ModuleList([lay[4] for lay in layers])
        sync = lambda: f8.sync_float8_amax_and_scale_history(model)
    flop_per_shape = {name: 3 * 2.0 * m * k * n for name, k, n, *_ in layers}
    flop_step = sum(flop_per_shape.values())
    # socket power with the tensors resident and nothing running, for the energy figures below
    torch.cuda.synchronize()
    time.sleep(0.5)
    idle = Telemetry()
    idle.start()
    time.sleep(0.3)
    idle_w = (idle.stop() or {}).get("socket_power_W_mean")

    if args.per_gemm_only is not None:
        print(json.dumps({"per_gemm_only": vendor_scaled_mm(torch, _native, layers, m, flop_step, max(2, args.steps), args.per_gemm_only),
                          "library_build_knobs": _native.build_knobs()}))
        return

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # ---- the timed region: K steps, every kernel launch bracketed by HIP events on its stream
    for _ in range(args.warmup):
        step(layers, sync=sync)
    torch.cuda.synchronize()
    _native.prof_reset()
    _native.prof_enable(True)
    telemetry = Telemetry()
    telemetry.start()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(layers, sync=sync)
    torch.cuda.synchronize()
    sec_step = (time.perf_counter() - t0) / args.steps
    telemetry = telemetry.stop()
    _native.prof_enable(False)
    prof = {name: _native.prof_read(kid) for name, kid in
            (("amax", _native.K_AMAX), ("cast", _native.K_CAST), ("gemm", _native.K_GEMM))}
    _native.prof_reset()

    n_gemm, ms_gemm, flop_gemm = prof["gemm"]
    gemm_tflops = flop_gemm / (ms_gemm * 1e-3) / 1e12 if ms_gemm > 0 else 0.0
    hbm = {}
    for kname in ("amax", "cast"):
        cnt, ms, nbytes = prof[kname]
        hbm[kname] = {"launches": cnt, "GB/s": nbytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0,
                      "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS if ms > 0 else 0.0,
                      "avg_ms": ms / max(cnt, 1), "algorithmic_GB_per_launch": nbytes / max(cnt, 1) / 1e9}

    if prof["amax"][1] > 0 and prof["cast"][1] > 0:  # dynamic scaling reads every tensor twice: both passes together
        both_bytes, both_ms = prof["amax"][2] + prof["cast"][2], prof["amax"][1] + prof["cast"][1]
        hbm["amax_plus_cast"] = {"GB/s": both_bytes / (both_ms * 1e-3) / 1e9,
                                 "frac_of_hbm_peak": both_bytes / (both_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                 "ms_per_step": both_ms / args.steps}
    traffic, traffic_note = gemm_traffic(m, args.scaling)

    # ---- per shape, and bf16 nn.Linear on the same GPU
    per_shape = {}
    for lay in layers:
        name = lay[0]
        one_sync = (lambda: f8.sync_float8_amax_and_scale_history(lay[4])) if sync is not None else None
        t = timed(torch, lambda: step([lay], sync=one_sync), max(2, args.steps // 2), 1)
        per_shape[name] = {"fp8_ms": t * 1e3, "fp8_TFLOP/s": flop_per_shape[name] / t / 1e12}
        # this shape's own kernels (the hbm_kernels figures above average over tensors of 134 MB to 1.9 GB)
        per_shape[name].update(_rates(_prof_window(torch, _native, lambda: step([lay], sync=one_sync), 2), reps=2))
    bf16_step = None
    if not args.no_bf16:
        for lay in layers:
            name = lay[0]
            t = timed(torch, lambda: step([lay], use_fp8=False), max(2, args.steps // 2), 1)
            per_shape[name]["bf16_ms"] = t * 1e3
            per_shape[name]["bf16_TFLOP/s"] = flop_per_shape[name] / t / 1e12
            per_shape[name]["speedup_vs_bf16"] = per_shape[name]["bf16_ms"] / per_shape[name]["fp8_ms"]
        bf16_step = sum(v["bf16_ms"] for v in per_shape.values()) * 1e-3

    # ---- the twelve GEMMs of a step alone, back to back on operands cast beforehand (untimed for `value`): what the
    # matrix-core kernel sustains, and the socket power and shader clock it runs at, without the cast phases in between
    gemm_loop = mfma_real = vendor = None
    if args.scaling == "dynamic":
        E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2
        ops = []
        for name, k, n, lin, mod, x, dy in layers:
            x8, _, sx = _native.cast_dynamic(x.detach(), E4, out_kblock=True)
            w8, _, sw = _native.cast_dynamic(lin.weight.detach(), E4, out_kblock=True)
            g8, _, sg = _native.cast_dynamic(dy, E5, out_kblock=True)
            ops.append((x8, sx, w8, sw, g8, sg))

        def gemms():
            for x8, sx, w8, sw, g8, sg in ops:
                if _native.tn_ok(m, x8.shape[0] * _native.KB, w8.shape[1]):
                    _native.gemm_nt_kb(x8, sx, w8, sw, torch.bfloat16)
                    _native.gemm_kb_ex(g8, False, sg, w8, True, sw, torch.bfloat16)
                    _native.gemm_kb_ex(g8, True, sg, x8, True, sx, torch.bfloat16)

        if all(_native.tn_ok(m, k, n) for _, k, n, *_ in layers):
            iters = max(8, 2 * args.steps)
            for _ in range(iters):  # untimed: power and clock settle over some hundred milliseconds
                gemms()
            torch.cuda.synchronize()
            tele = Telemetry()
            tele.start()
            t0 = time.perf_counter()
            for _ in range(iters):
                gemms()
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) / iters
            gemm_loop = {"TFLOP/s": flop_step / dt / 1e12, "frac_of_fp8_peak": flop_step / dt / 1e12 / PEAK_FP8_TFLOPS,
                         "ms_per_12_gemms": dt * 1e3, "iterations": iters, "telemetry": tele.stop()}
            if gemm_loop["telemetry"] and idle_w:
                # joules per flop on top of what the idle socket draws: under the power cap this, not the number of
                # stalled cycles, is what sets the rate
                gemm_loop["idle_socket_power_W"] = idle_w
                gemm_loop["pJ_per_flop_above_idle"] = (gemm_loop["telemetry"]["socket_power_W_mean"] - idle_w) / gemm_loop["TFLOP/s"]
        # the same register-only loop on the fp8 bytes the benchmark's GEMMs actually multiply (x8 of the first shape)
        mfma_real = probe_mfma(torch, True, operands=ops[0][0], idle_w=idle_w, order=args.mfma_order)
        del ops
        vendor = vendor_scaled_mm(torch, _native, layers, m, flop_step, max(4, args.steps))

    # the matrix cores' own ceiling on this box: register-only MFMA loop, clock-limited (zeros) and power-limited (random bytes)
    mfma_zero = probe_mfma(torch, False, idle_w=idle_w, order=args.mfma_order)
    mfma_random = probe_mfma(torch, True, idle_w=idle_w, order=args.mfma_order)

    out = {
        "metric": "Float8Linear fwd+bwd TFLOP/s at LLaMa-2-70B shapes (1 GPU); cast GB/s",
        "value": flop_step / sec_step / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8",
        "data": "synthetic",
        "config": {
            "workload": f"LLaMa-2-70B linear shapes, {args.scaling} scaling, M={m} tokens bf16, (K->N) 8192->10240, 8192->8192, "
                        "8192->57344, 28672->8192; fwd+bwd with dY ~N(0,1e-2); one step = all four shapes",
            "flop_per_step": flop_step,
            "flop_convention": "3 * 2*M*K*N per shape",
        },
        "roofline": {
            "kernel": "f8mi gemm_nt_dma16_kernel (fp8 MFMA GEMM on k-blocked operands, read as they lie or transposed; all 12 launches of a step)",
            "bound": "mfma",
            "achieved": gemm_tflops,
            "peak": PEAK_FP8_TFLOPS,
            "unit": "TFLOP/s",
            "frac": gemm_tflops / PEAK_FP8_TFLOPS,
            "traffic": traffic,
            "traffic_unit": traffic_note,
            "launches": n_gemm,
            "avg_launch_ms": ms_gemm / max(n_gemm, 1),
            "flop_per_launch": flop_gemm / max(n_gemm, 1),
            "mfma_only_zero_operands": mfma_zero,
            "mfma_only_random_operands": mfma_random,
            "mfma_only_benchmark_operands": mfma_real,
            "frac_of_mfma_only_random": gemm_tflops / mfma_random["TFLOP/s"] if mfma_random else None,
            "gemms_back_to_back": gemm_loop,
            "vendor_scaled_mm": vendor,
        },
        "telemetry": telemetry,
        "hbm_kernels": hbm,
        "per_shape": per_shape,
        "frac_of_fp8_peak_end_to_end": flop_step / sec_step / 1e12 / PEAK_FP8_TFLOPS,
    }
    out["library_build_knobs"] = _native.build_knobs()  # "" = the library as shipped
    if not args.no_other_configs:
        out["other_configs"] = other_configs(torch, f8, _native, layers, args)
    if bf16_step:
        out["bf16_linear"] = {"ms_per_step": bf16_step * 1e3, "TFLOP/s": flop_step / bf16_step / 1e12,
                              "speedup_fp8_over_bf16": bf16_step / sum(v["fp8_ms"] * 1e-3 for v in per_shape.values())}
    if not args.no_cpu_baseline:
        # free the GPU-side tensors' host shadows are none; the CPU leg only needs host memory
        out["cpu_baseline"] = cpu_baseline(torch, args.cpu_seconds)
        out["cpu_baseline"]["host"] = {"cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads(),
                                       "torch": torch.__version__}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
