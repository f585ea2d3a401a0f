#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Step = one pass of the FLUX.1 single-stream block's quantized linears at
1024x1024 (the configuration the headline metric is quoted on): x[4608,3072] @ W4[21504,3072]^T followed by
x2[4608,15360] @ W4[3072,15360]^T, group size 64, bf16 activations, synthetic
N(0,1) activations and N(0,0.02) weights quantized on the device by this
library.  Prints ONE JSON line; `value` is TFLOP/s over the two GEMMs with all
operands resident in HBM.

The same line carries
  roofline     - the W4A16 GEMM kernel against the dense bf16 MFMA peak, from
                 HIP-event timing of the launches in the timed region;
  secondary    - the W8 (and W4) dequant-GEMV (adaLN modulation shape, M=1 and
                 M=4) against the HBM peak, weights rotated through > 256 MB so
                 the memory-side cache cannot serve them; the quantize/pack
                 pass over both block weights; the text-stream shapes (M=512)
                 of a joint block; and, for comparison, the BLAS library's
                 plain bf16 GEMM on the step's own activations and dequantised
                 weights;
  cpu_baseline - the CPU oracle's scalar qmm (a port of MLX's CPU loop; MLX
                 itself cannot be installed here) on a bounded row sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

# L2 <-> fabric bytes per launch are hardware counters (rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE, scaled by a plain copy of known size) and cannot be read from inside
# this script: `roofline.traffic` is taken from the line `traffic_bytes_per_launch:
# <number>` of the committed summary of that profile, and says so.
TRAFFIC_PROFILES = {
    "gemm": "profiles/qmm_w4a16_flux_single_block_m4608.md",
    "gemv": "profiles/qmv_w8_adaln_3072x18432.md",
}

M_TOKENS = 4608
CONFIG = 3  # the benchmark configuration of the step: seeds are 1000 * config + tensor index
LINEARS = (("linear1", 3072, 21504), ("linear2", 15360, 3072))  # (name, K, N)
GS, BITS = 64, 4


def qmm_bytes(M, K, N, bits, bias=False):
    return N * K * bits // 8 + 4 * N * K // 64 + 2 * M * K + 2 * M * N + (2 * N if bias else 0)


def quantize_bytes(N, K, bits):
    return 2 * N * K + N * K * bits // 8 + 4 * N * K // 64


def profiled_traffic(which):
    """(bytes per launch, source) from the committed counter profile, or (None, reason)."""
    path = os.path.join(ROOT, TRAFFIC_PROFILES[which])
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1].split()[0]), (
                        f"{TRAFFIC_PROFILES[which]} (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE of an earlier run of "
                        "this command, scaled by a 256 MiB copy; not counted in this run)")
    except OSError:
        pass
    return None, f"{TRAFFIC_PROFILES[which]} holds no traffic_bytes_per_launch line"


def seeded_bf16(torch, dev, config, index, shape, std):
    """The benchmark's input convention: numpy default_rng(1000 * config + index),
    float32 normals scaled by std, rounded once to bfloat16."""
    import numpy as np

    rng = np.random.default_rng(1000 * config + index)
    a = rng.standard_normal(shape, dtype=np.float32)
    if std != 1.0:
        a *= np.float32(std)
    return torch.from_numpy(a).to(dev).to(torch.bfloat16)


class Telemetry:
    """Socket power and shader clock of GPU 0 sampled from sysfs by a thread
    while a timed region runs (ordinary user, nothing is changed)."""

    def __init__(self, period=0.01):
        import glob

        self.period = period
        hw = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))
        self.power = next((os.path.join(d, f) for d in hw for f in ("power1_average", "power1_input")
                           if os.path.exists(os.path.join(d, f))), None)
        self.cap = next((os.path.join(d, "power1_cap") for d in hw if os.path.exists(os.path.join(d, "power1_cap"))),
                        None)
        sclk = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.sclk = sclk[0] if sclk else None
        self.samples = []

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                return f.read()
        except OSError:
            return None

    def _sample(self):
        watts = mhz = None
        txt = self._read(self.power) if self.power else None
        if txt:
            watts = int(txt) / 1e6
        txt = self._read(self.sclk) if self.sclk else None
        for line in (txt or "").splitlines():
            if line.rstrip().endswith("*"):
                digits = "".join(ch for ch in line.split(":", 1)[1] if ch.isdigit())
                mhz = int(digits) if digits else None
        return watts, mhz

    def __enter__(self):
        import threading

        self._stop = threading.Event()

        def run():
            while not self._stop.is_set():
                self.samples.append(self._sample())
                self._stop.wait(self.period)

        self._thread = threading.Thread(target=run, daemon=True)
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join()

    def summary(self):
        watts = [w for w, _ in self.samples if w is not None]
        mhz = [m for _, m in self.samples if m is not None]
        cap = self._read(self.cap) if self.cap else None
        return {
            "samples": len(self.samples),
            "socket_power_w_mean": round(sum(watts) / len(watts), 1) if watts else None,
            "socket_power_w_max": round(max(watts), 1) if watts else None,
            "power_cap_w": int(cap) / 1e6 if cap else None,
            "sclk_mhz_mean": round(sum(mhz) / len(mhz), 1) if mhz else None,
            "sclk_mhz_min": min(mhz) if mhz else None,
            "source": "sysfs hwmon power1 and pp_dpm_sclk of card 0, sampled every 10 ms",
        }


def event_ms(fn, iters, torch):
    """Average milliseconds per call of fn over `iters` back-to-back calls,
    measured with HIP events on the current stream (the stream fn launches on)."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def graph_ms(fn, calls, replays, torch):
    """Average milliseconds per call of fn with `calls` calls captured into one
    HIP graph and replayed `replays` times: back-to-back kernels without the
    host's per-call launch cost, which would otherwise dominate a ~10 us kernel.
    Events are recorded on the stream the graph replays on."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(calls):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        graph.replay()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / (calls * replays)


def cpu_baseline(torch, x, wq, s, b, sample_rows):
    """Times the oracle's scalar qmm_t (float32 accumulation) on the first
    `sample_rows` rows of the linear1 problem, on all host threads and on one."""
    import numpy as np
    from oracle import mlx_affine as o

    def raw16(t):
        return t.contiguous().cpu().view(torch.int16).numpy().view(np.uint16)

    xs = raw16(x[:sample_rows])
    wq_h = wq.cpu().view(torch.int32).numpy().view(np.uint32)
    s_h, b_h = raw16(s), raw16(b)
    N, K = wq_h.shape[0], xs.shape[1]
    threads = min(o.num_threads(), len(os.sched_getaffinity(0)))
    flops = 2.0 * sample_rows * N * K
    t0 = time.perf_counter()
    o.c_qmm_t(xs, o.BF16, wq_h, s_h, b_h, o.BF16, None, GS, BITS, threads=threads)
    t_all = time.perf_counter() - t0
    one_rows = max(1, min(64, sample_rows // 8))
    t0 = time.perf_counter()
    o.c_qmm_t(xs[:one_rows], o.BF16, wq_h, s_h, b_h, o.BF16, None, GS, BITS, threads=1)
    t_one = time.perf_counter() - t0
    return {
        "value": round(flops / t_all / 1e12, 6),
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"first {sample_rows} of {M_TOKENS} rows of linear1 (K=3072, N=21504, W4 gs64), "
                  f"{t_all:.1f} s on {threads} threads; scalar float32-accumulating port of MLX's CPU _qmm_t "
                  "(MLX is not installable offline)",
        "single_thread_value": round(2.0 * one_rows * N * K / t_one / 1e12, 6),
        "single_thread_sample": f"first {one_rows} rows, {t_one:.1f} s on 1 thread",
    }


# (configuration, M, K, N, bits) of every GEMM of BASELINE.json's configurations (the matvecs are the bench's own leg)
CONFIG_SHAPES = (
    ("1 FLUX to_q", 4096, 3072, 3072, 4),
    ("3 FLUX single block linear1", 4608, 3072, 21504, 4), ("3 FLUX single block linear2", 4608, 15360, 3072, 4),
    ("4 Z-Image", 4352, 3840, 3840, 8), ("4 Z-Image", 4352, 3840, 10240, 8), ("4 Z-Image", 4352, 10240, 3840, 8),
    ("5 Qwen-Image image stream", 6889, 3072, 3072, 4), ("5 Qwen-Image image stream", 6889, 3072, 12288, 4),
    ("5 Qwen-Image image stream", 6889, 12288, 3072, 4),
    ("5 Qwen-Image text stream", 256, 3072, 3072, 4), ("5 Qwen-Image text stream", 256, 3072, 12288, 4),
    ("5 Qwen-Image text stream", 256, 12288, 3072, 4),
    ("text stream at M = 512", 512, 3072, 3072, 4), ("text stream at M = 512", 512, 3072, 12288, 4),
    ("text stream at M = 512", 512, 12288, 3072, 4),
)


def config_table(torch, mflux_amd, dev):
    """Per shape: 100 calls of quantized_matmul back to back, then 100 of torch.matmul
    on the dequantised weights, each timed as a whole with HIP events (sustained,
    unlike a short burst; under `rocprofv3 --kernel-trace --stats` the same run
    gives every kernel's own average)."""
    rows = []
    for name, M, K, N, bits in CONFIG_SHAPES:
        x = seeded_bf16(torch, dev, 3, 0, (M, K), 1.0)
        w = seeded_bf16(torch, dev, 3, 1, (N, K), 0.02)
        wq, s, b = mflux_amd.quantize(w, GS, bits)
        w16 = mflux_amd.dequantize(wq, s, b, GS, bits)
        del w
        row = {"config": name, "M": M, "K": K, "N": N, "bits": bits}
        for key, fn in (("mfq", lambda: mflux_amd.quantized_matmul(x, wq, s, b, group_size=GS, bits=bits)),
                        ("library_bf16", lambda: torch.matmul(x, w16.t()))):
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
            ms = event_ms(fn, 100, torch)
            row[key] = {"us": round(ms * 1e3, 1), "tflops": round(2.0 * M * K * N / ms / 1e9, 1)}
        rows.append(row)
        del x, wq, s, b, w16
    return {"workload": "GEMM shapes of the BASELINE configurations, 100 calls each back to back", "rows": rows}


def baseline_configs(torch, mflux_amd, dev, quick=False):
    """BASELINE configurations 1, 4 and 5 as wholes (the headline is configuration 3, the matvec
    leg configuration 2): the summed time of a configuration's quantized linears, calls back to
    back on one stream with HIP events around them, and 2MNK of its GEMMs over that time against
    the dense bf16 peak.  Configuration 5 keeps all 60 blocks' weights resident (11.5 GB of packed
    4-bit codes, scales and biases, every block its own tensors) and visits them in order, so a
    block's weights are cold when its linears run; its two modulation matvecs per block are in the
    time and not in the FLOPs."""
    from mflux_amd import nn as qnn

    def qlinear(config, index, K, N, bits, bias, w=None):
        lin = qnn.QuantizedLinear(K, N, bias=bias, group_size=GS, bits=bits)
        if w is None:
            w = seeded_bf16(torch, dev, config, index, (N, K), 0.02)
        lin.weight, lin.scales, lin.biases = mflux_amd.quantize(w, GS, bits)
        if bias:
            lin.bias = seeded_bf16(torch, dev, config, index + 500, (N,), 0.02)
        return lin

    def timed(fn, warm, iters):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        return event_ms(fn, iters, torch)

    out = {}
    # -- 1: FLUX.1 to_q, 4096 x 3072 -> 3072, W4, bias
    x = seeded_bf16(torch, dev, 1, 0, (4096, 3072), 1.0)
    lin = qlinear(1, 1, 3072, 3072, 4, True)
    ms = timed(lambda: lin(x), 10, 50)
    flops = 2.0 * 4096 * 3072 * 3072
    out["config1_flux_to_q_m4096_w4"] = {"us": round(ms * 1e3, 1), "tflops": round(flops / ms / 1e9, 1),
                                         "frac_mfma": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    # the same layer with its 16-bit copy kept (QuantizedLinear.prepare(): 2 bytes per weight held, the call is
    # the GEMM alone): a variant beside the configuration's figure, not instead of it
    lin.prepare()
    ms = timed(lambda: lin(x), 10, 50)
    out["config1_flux_to_q_m4096_w4"]["with_kept_copy"] = {
        "us": round(ms * 1e3, 1), "tflops": round(flops / ms / 1e9, 1),
        "frac_mfma": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    del lin, x

    # -- 4: Z-Image block, M = 4352, hidden 3840, W8, no bias: q, k, v, out, w1, w3, w2
    M4 = 4352
    x = seeded_bf16(torch, dev, 4, 0, (M4, 3840), 1.0)
    xh = seeded_bf16(torch, dev, 4, 1, (M4, 10240), 1.0)
    q, k, v, o = (qlinear(4, 10 + i, 3840, 3840, 8, False) for i in range(4))
    w1, w3 = (qlinear(4, 20 + i, 3840, 10240, 8, False) for i in range(2))
    w2 = qlinear(4, 30, 10240, 3840, 8, False)
    flops = 2.0 * M4 * (4 * 3840 * 3840 + 3 * 3840 * 10240)

    def separate():
        q(x), k(x), v(x), o(x), w1(x), w3(x), w2(xh)

    qkv = qnn.concat_quantized([q, k, v])
    gate_up = qnn.stack_gate_up(w1, w3)

    def fused():  # q/k/v as one linear; silu(w1 x) * w3 x in the epilogue of one linear over the stacked pair
        qkv(x), o(x), qnn.swiglu_linear(gate_up, x), w2(xh)

    res = {}
    for key, fn in (("seven_calls", separate), ("qkv_as_one_and_swiglu_epilogue", fused)):
        ms = timed(fn, 5, 20)
        res[key] = {"us": round(ms * 1e3, 1), "tflops": round(flops / ms / 1e9, 1),
                    "frac_mfma": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    held = sum(int(layer.prepare()) * 2 * layer.output_dims * layer.input_dims for layer in (q, k, v, o, w1, w3, w2))
    ms = timed(separate, 5, 20)
    res["seven_calls_with_kept_copies"] = {"us": round(ms * 1e3, 1), "tflops": round(flops / ms / 1e9, 1),
                                           "frac_mfma": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                                           "copies_held_gb": round(held / 1e9, 2)}
    out["config4_zimage_block_m4352_w8"] = res
    del q, k, v, o, w1, w3, w2, qkv, gate_up, x, xh

    # -- 5: Qwen-Image step, 60 blocks, image stream 6889 tokens, text stream 256, W4, bias
    n_blocks = 6 if quick else 60
    Mi, Mt = 6889, 256
    xi, xt = seeded_bf16(torch, dev, 5, 0, (Mi, 3072), 1.0), seeded_bf16(torch, dev, 5, 1, (Mt, 3072), 1.0)
    xih, xth = seeded_bf16(torch, dev, 5, 2, (Mi, 12288), 1.0), seeded_bf16(torch, dev, 5, 3, (Mt, 12288), 1.0)
    temb = seeded_bf16(torch, dev, 5, 4, (1, 3072), 1.0)
    base = {(3072, 3072): seeded_bf16(torch, dev, 5, 10, (3072, 3072), 0.02),
            (3072, 12288): seeded_bf16(torch, dev, 5, 11, (12288, 3072), 0.02),
            (12288, 3072): seeded_bf16(torch, dev, 5, 12, (3072, 12288), 0.02),
            (3072, 18432): seeded_bf16(torch, dev, 5, 13, (18432, 3072), 0.02)}
    blocks = []
    for bi in range(n_blocks):
        def lin(K, N, shift):  # every linear its own weights: the seeded matrix of its shape, rows rotated
            return qlinear(5, 0, K, N, 4, True, w=torch.roll(base[(K, N)], shifts=7 * (16 * bi + shift) + 1, dims=0))
        streams = []
        for st in range(2):
            attn = [lin(3072, 3072, 8 * st + i) for i in range(4)]
            streams.append({"q": attn[0], "k": attn[1], "v": attn[2], "out": attn[3],
                            "qkv": qnn.concat_quantized(attn[:3], share_storage=True),
                            "mlp_in": lin(3072, 12288, 8 * st + 4), "mlp_out": lin(12288, 3072, 8 * st + 5),
                            "mod": lin(3072, 18432, 8 * st + 6)})
        blocks.append(streams)
    del base
    resident = sum(t.numel() * t.element_size() for streams in blocks for s_ in streams
                   for key in ("qkv", "out", "mlp_in", "mlp_out", "mod")
                   for t in (s_[key].weight, s_[key].scales, s_[key].biases))
    flops = n_blocks * 2.0 * (Mi + Mt) * (4 * 3072 * 3072 + 2 * 3072 * 12288)

    def step_separate():
        for streams in blocks:
            for s_, x_, xh_ in ((streams[0], xi, xih), (streams[1], xt, xth)):
                qnn.silu_linear(s_["mod"], temb)
                s_["q"](x_), s_["k"](x_), s_["v"](x_), s_["out"](x_), s_["mlp_in"](x_), s_["mlp_out"](xh_)

    def step_fused():  # q/k/v as one linear
        for streams in blocks:
            for s_, x_, xh_ in ((streams[0], xi, xih), (streams[1], xt, xth)):
                qnn.silu_linear(s_["mod"], temb)
                s_["qkv"](x_), s_["out"](x_), s_["mlp_in"](x_), s_["mlp_out"](xh_)

    # the same calls with the two streams of tokens on two HIP streams: a block's text-stream linears and
    # modulation matvecs need nothing from its image-stream linears (the streams meet in the attention, which
    # is not part of this configuration), and run on the compute units that the image stream's short last
    # round of tiles leaves idle
    side = torch.cuda.Stream()

    def step_two_streams():
        main = torch.cuda.current_stream()
        side.wait_stream(main)
        with torch.cuda.stream(side):
            for streams in blocks:
                s_ = streams[1]
                qnn.silu_linear(s_["mod"], temb), qnn.silu_linear(streams[0]["mod"], temb)
                s_["qkv"](xt), s_["out"](xt), s_["mlp_in"](xt), s_["mlp_out"](xth)
        for streams in blocks:
            s_ = streams[0]
            s_["qkv"](xi), s_["out"](xi), s_["mlp_in"](xi), s_["mlp_out"](xih)
        main.wait_stream(side)

    res = {"blocks": n_blocks, "weights_resident_gb": round(resident / 1e9, 2)}
    for key, fn in (("sixteen_calls_per_block", step_separate), ("qkv_as_one", step_fused),
                    ("qkv_as_one_and_text_stream_on_a_second_hip_stream", step_two_streams)):
        ms = timed(fn, 1, 2 if not quick else 1)
        res[key] = {"ms_per_step": round(ms, 2), "tflops": round(flops / ms / 1e9, 1),
                    "frac_mfma": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    # the image stream's linears with their 16-bit copies kept (13.6 GB more for the 60 blocks; the text stream's
    # 256 rows do not use one)
    held = 0
    for streams in blocks:
        for key in ("qkv", "out", "mlp_in", "mlp_out"):
            layer = streams[0][key]
            held += int(layer.prepare()) * 2 * layer.output_dims * layer.input_dims
    ms = timed(step_two_streams, 1, 2 if not quick else 1)
    res["qkv_as_one_two_hip_streams_and_kept_copies"] = {
        "ms_per_step": round(ms, 2), "tflops": round(flops / ms / 1e9, 1),
        "frac_mfma": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4), "copies_held_gb": round(held / 1e9, 2)}
    # ... and the 120 modulation linears of the step (they all take the same silu(temb)) as one matvec over their
    # stacked rows at the start of the step (nn.concat_quantized(share_storage=True): the layers become views)
    mods = qnn.concat_quantized([s_["mod"] for streams in blocks for s_ in streams], share_storage=True)

    def step_two_streams_one_modulation():
        main = torch.cuda.current_stream()
        side.wait_stream(main)
        with torch.cuda.stream(side):
            qnn.silu_linear(mods, temb)
            for streams in blocks:
                s_ = streams[1]
                s_["qkv"](xt), s_["out"](xt), s_["mlp_in"](xt), s_["mlp_out"](xth)
        for streams in blocks:
            s_ = streams[0]
            s_["qkv"](xi), s_["out"](xi), s_["mlp_in"](xi), s_["mlp_out"](xih)
        main.wait_stream(side)

    ms = timed(step_two_streams_one_modulation, 1, 2 if not quick else 1)
    res["qkv_as_one_two_hip_streams_kept_copies_and_one_modulation_call"] = {
        "ms_per_step": round(ms, 2), "tflops": round(flops / ms / 1e9, 1),
        "frac_mfma": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    out["config5_qwen_image_step_w4"] = res
    del blocks, mods
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sustain-s", type=float, default=1.5,
                    help="seconds the step keeps running behind the timed region while socket power and "
                         "shader clock are sampled (0: skip)")
    ap.add_argument("--cpu-sample-rows", type=int, default=2304)
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the GEMV and quantize measurements (they replay HIP graphs)")
    ap.add_argument("--configs-quick", action="store_true",
                    help="the Qwen-Image leg of secondary.configs on 6 blocks instead of 60 (for profiling runs)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one plain 256 MiB device-to-device copy, the known-size kernel that "
                         "FETCH_SIZE / WRITE_SIZE counter readings are scaled by")
    ap.add_argument("--config-table", action="store_true",
                    help="instead of the benchmark: every GEMM shape of the BASELINE configurations, each 100 calls "
                         "back to back (for a kernel trace), with the BLAS library's bf16 GEMM on the dequantised "
                         "weights beside it; prints one JSON object")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (--gpus 1); nothing is sharded across devices")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device visible")
    import mflux_amd

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(3000)  # for the side legs only; the step's operands are seeded by numpy

    if args.config_table:
        print(json.dumps(config_table(torch, mflux_amd, dev)))
        return

    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(7)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- operands of the step, resident in HBM --------------------------------
    ops = []
    quant_ms = {}
    for lin, (name, K, N) in enumerate(LINEARS):
        x = seeded_bf16(torch, dev, CONFIG, 10 * lin + 0, (M_TOKENS, K), 1.0)
        w = seeded_bf16(torch, dev, CONFIG, 10 * lin + 1, (N, K), 0.02)
        wq, s, b = mflux_amd.quantize(w, GS, BITS)
        copies = [w] + [w.clone() for _ in range(3)]  # > 256 MB in rotation: cold reads
        turn = {"i": 0}

        def quantize_call():
            turn["i"] += 1
            mflux_amd.quantize(copies[turn["i"] % len(copies)], GS, BITS)

        if not args.no_secondary:
            quant_ms[name] = graph_ms(quantize_call, 8, 5, torch)
        del copies, w
        ops.append((name, x, wq, s, b))

    def step():
        for _, x, wq, s, b in ops:
            mflux_amd.quantized_matmul(x, wq, s, b, group_size=GS, bits=BITS)

    # ---- secondary legs on the step's own operands (they run first: the headline below is then timed on a
    # chip that is already under matrix load, with exactly the requested warm-up steps in front of it) -----
    #   the library's bf16 GEMM on the same operands
    library = {}
    for name, x, wq, s, b in (() if args.no_secondary else ops):
        w16 = mflux_amd.dequantize(wq, s, b, group_size=GS, bits=BITS)
        for _ in range(5):  # the library picks and caches its kernel on the first calls
            torch.matmul(x, w16.t())
        torch.cuda.synchronize()
        ms = event_ms(lambda: torch.matmul(x, w16.t()), 20, torch)
        K, N = x.shape[1], wq.shape[0]
        library[name] = {"us": round(ms * 1e3, 1), "tflops": round(2.0 * M_TOKENS * K * N / ms / 1e9, 1)}
        del w16
    #   the same linears on a prepared copy of their weights (the 16-bit copy made once instead of on every
    #   call, 2 bytes per weight held: the GEMM kernel alone)
    prepared = {}
    for name, x, wq, s, b in (() if args.no_secondary else ops):
        K, N = x.shape[1], wq.shape[0]
        copy = mflux_amd.prepare_weights(wq, s, b, group_size=GS, bits=BITS)
        for _ in range(3):
            mflux_amd.quantized_matmul_prepared(x, copy, N)
        torch.cuda.synchronize()
        ms = event_ms(lambda: mflux_amd.quantized_matmul_prepared(x, copy, N), 20, torch)
        prepared[name] = {"us": round(ms * 1e3, 1), "tflops": round(2.0 * M_TOKENS * K * N / ms / 1e9, 1),
                          "copy_mb_held": round(copy.numel() / 1e6, 1)}
        del copy

    # ---- the headline: args.warmup untimed steps, then exactly args.steps timed ones ------------------
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    kernel_ms_per_step = start.elapsed_time(stop) / args.steps
    # Beside it, not in `value`: the same step once batches of ten agree within 1 % (the chip takes
    # some hundred launches under load before clocks and power settle), and its first batches.
    settle, prev = [], None
    for _ in range(40):
        ms = event_ms(step, 10, torch)
        settle.append(round(ms, 4))
        if prev is not None and abs(ms - prev) <= 0.01 * prev:
            break
        prev = ms
    settled_ms = event_ms(step, args.steps, torch)
    # The power sensor is a moving average that needs about half a second to follow the load, far
    # longer than the timed region above: the same step therefore runs on for args.sustain_s
    # seconds right behind it, and power and clock are the samples of the second half of that leg.
    sustained = None
    if args.sustain_s > 0:
        n_sus = max(10, int(args.sustain_s * 1e3 / kernel_ms_per_step))
        with Telemetry() as telemetry:
            ms = event_ms(step, n_sus, torch)
        telemetry.samples = telemetry.samples[len(telemetry.samples) // 2:]
        sustained = {"steps": n_sus, "ms_per_step": round(ms, 4),
                     "tflops": round(sum(2.0 * M_TOKENS * K * N for _, K, N in LINEARS) / ms / 1e9, 1),
                     **telemetry.summary()}

    flops = sum(2.0 * M_TOKENS * K * N for _, K, N in LINEARS)
    value = flops / (ms_per_step * 1e-3) / 1e12
    launches = len(LINEARS)
    achieved = flops / (kernel_ms_per_step * 1e-3) / 1e12  # = mean flops per launch / mean launch duration
    traffic, traffic_source = profiled_traffic("gemm")
    roofline = {
        # one call = two launches on this shape: the 16-bit copy of the dequantised weights, then the GEMM on it;
        # `achieved` is the call's algorithmic 2MNK over both, so the GEMM kernel alone sits above it
        # (profiles/ holds each kernel's own average)
        "kernel": "frag_gemm_kernel<BF16> behind dequant_frag_kernel<BF16,64,4> (both launches of a call)",
        "launches_per_call": 2,
        "bound": "mfma",
        "achieved": round(achieved, 2),
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
        "traffic": traffic,
        "traffic_source": traffic_source,
        "avg_launch_us": round(kernel_ms_per_step * 1e3 / launches, 2),
        "flops_per_launch": flops / launches,
        "sustained": sustained,
        "timed_region": f"{args.warmup} warm-up steps, then {args.steps} timed steps, right behind the "
                        "library-GEMM and prepared-copy legs on the same operands",
        "settled": {"ms_per_step": round(settled_ms, 4), "tflops": round(flops / settled_ms / 1e9, 1),
                    "frac": round(flops / settled_ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                    "batches_of_ten_until_two_agree_ms": settle},
    }

    # per-shape GEMM timings
    per_shape = {}
    for name, x, wq, s, b in ops:
        ms = event_ms(lambda: mflux_amd.quantized_matmul(x, wq, s, b, group_size=GS, bits=BITS), 20, torch)
        K, N = x.shape[1], wq.shape[0]
        per_shape[name] = {"us": round(ms * 1e3, 1), "tflops": round(2.0 * M_TOKENS * K * N / ms / 1e9, 1)}

    # ---- secondary: a rank-16 LoRA on the two linears --------------------------
    # the whole layer (x @ A included) as one fused call against the reference's
    # composition of separate matmuls, and the kernel alone with the update
    lora = {}
    for name, x, wq, s, b in (() if args.no_secondary else ops):
        from mflux_amd.lora import LoRALinear, _composed, pack_adapters

        K, N = x.shape[1], wq.shape[0]
        base = mflux_amd.nn.QuantizedLinear(K, N, bias=False, group_size=GS, bits=BITS)
        base.weight, base.scales, base.biases = wq, s, b
        layer = LoRALinear.from_linear(base, r=16, scale=1.0)
        with torch.no_grad():
            a_cat, bs = pack_adapters([layer], torch.bfloat16)
            t = torch.matmul(x, a_cat)
            calls = {
                "kernel_with_update_us": lambda: mflux_amd.quantized_matmul(x, wq, s, b, group_size=GS, bits=BITS,
                                                                            low_rank=(t, bs)),
                "fused_layer_us": lambda: layer(x),
                "separate_matmuls_us": lambda: _composed(base, [layer], x),
            }
            for fn in calls.values():
                for _ in range(5):
                    fn()
            best = {key: float("inf") for key in calls}
            for _ in range(3):  # the three variants in turn, so that clock drift touches them alike
                for key, fn in calls.items():
                    best[key] = min(best[key], event_ms(fn, 10, torch))
            res = {key: round(ms * 1e3, 1) for key, ms in best.items()}
        res["base_us"] = per_shape[name]["us"]
        lora[name] = res
        del base, layer, a_cat, bs, t

    # ---- secondary: GEMV of the adaLN modulation shape, cold weights -----------
    gemv = {}
    Kg, Ng = 3072, 18432
    # configuration 2: W ~ N(0, 0.02) [18432, 3072], eight different matrices (seeds 2001..2008) so that the
    # weights in rotation exceed the 256 MB memory-side cache; at 4 bits the eight are stored twice
    gemv_w16 = [] if args.no_secondary else [seeded_bf16(torch, dev, 2, 1 + i, (Ng, Kg), 0.02) for i in range(8)]
    for bits_g in (() if args.no_secondary else (8, 4)):
        bufs = [mflux_amd.quantize(w, GS, bits_g) for w in gemv_w16]
        if bits_g == 4:
            bufs += [tuple(t.clone() for t in buf) for buf in bufs]
        n_buf = len(bufs)  # more than 256 MB in rotation
        bias = seeded_bf16(torch, dev, 2, 100, (Ng,), 0.02)
        res = {}
        for Mg in (1, 4):
            temb = seeded_bf16(torch, dev, 2, 0, (Mg, Kg), 1.0)
            xg = mflux_amd.silu(temb)  # x = SiLU(temb), evaluated as MLX's nn.silu does on bfloat16
            state = {"i": 0}

            def gemv_call():
                wqg, sg, bg = bufs[state["i"] % n_buf]
                state["i"] += 1
                mflux_amd.quantized_matmul(xg, wqg, sg, bg, group_size=GS, bits=bits_g, bias=bias)

            ms = graph_ms(gemv_call, 4 * n_buf, 10, torch)
            nbytes = qmm_bytes(Mg, Kg, Ng, bits_g, bias=True)
            gbs = nbytes / (ms * 1e-3) / 1e9
            res[f"M{Mg}"] = {"us": round(ms * 1e3, 2), "GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4),
                             "bytes": nbytes,
                             "weights": f"rotating over {n_buf} buffers ({n_buf * Ng * Kg * bits_g // 8 >> 20} MiB)"}
        # the whole modulation call linear(silu(temb)) at M = 1: the activation inside the matvec
        # kernel against an elementwise pass in front of it (what the reference runs)
        temb16 = seeded_bf16(torch, dev, 2, 0, (1, Kg), 1.0)
        state = {"i": 0}

        def fused_call():
            wqg, sg, bg = bufs[state["i"] % n_buf]
            state["i"] += 1
            mflux_amd.silu_quantized_matmul(temb16, wqg, sg, bg, group_size=GS, bits=bits_g, bias=bias)

        def separate_call():
            wqg, sg, bg = bufs[state["i"] % n_buf]
            state["i"] += 1
            mflux_amd.quantized_matmul(mflux_amd.silu(temb16), wqg, sg, bg, group_size=GS, bits=bits_g, bias=bias)

        # all modulation linears of a step as one call: they all take the same silu(temb), so their packed
        # weights stack along N.  W8: the 38 linears of FLUX.1's double blocks (2.3 GB); W4: the 120 of
        # Qwen-Image's 60 blocks (3.8 GB).  Cold by size.
        n_stack = 38 if bits_g == 8 else 120
        picks = [bufs[i % n_buf] for i in range(n_stack)]
        wq_all, s_all, b_all = (torch.cat([p[j] for p in picks]) for j in range(3))
        bias_all = bias.repeat(n_stack)
        call_all = lambda: mflux_amd.silu_quantized_matmul(temb16, wq_all, s_all, b_all, group_size=GS,
                                                           bits=bits_g, bias=bias_all)
        call_all()
        ms = event_ms(call_all, 10, torch)
        nbytes = qmm_bytes(1, Kg, n_stack * Ng, bits_g, bias=True)
        res[f"M1_{n_stack}_linears_one_call"] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1),
                                                 "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                                                 "bytes": nbytes}
        del picks, wq_all, s_all, b_all, bias_all
        # the two modulation linears of ONE joint block (norm1 and norm1_context take the same text_embeddings,
        # src/mflux/models/flux/model/flux_transformer/joint_transformer_block.py:29-38) as one call, pairs of
        # weights in rotation: the smallest stack a block offers
        pairs = [tuple(torch.cat([bufs[(2 * i) % n_buf][j], bufs[(2 * i + 1) % n_buf][j]]) for j in range(3))
                 for i in range(n_buf // 2)]
        bias_pair = bias.repeat(2)
        state = {"i": 0}

        def pair_call():
            wqg, sg, bg = pairs[state["i"] % len(pairs)]
            state["i"] += 1
            mflux_amd.silu_quantized_matmul(temb16, wqg, sg, bg, group_size=GS, bits=bits_g, bias=bias_pair)

        ms = graph_ms(pair_call, 4 * len(pairs), 10, torch)
        nbytes = qmm_bytes(1, Kg, 2 * Ng, bits_g, bias=True)
        res["M1_2_linears_of_a_block_one_call"] = {"us": round(ms * 1e3, 2), "GB/s": round(nbytes / ms / 1e6, 1),
                                                   "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                                                   "bytes": nbytes}
        del pairs, bias_pair
        res["M1_with_silu"] = {"fused_us": round(graph_ms(fused_call, 4 * n_buf, 10, torch) * 1e3, 2),
                               "separate_us": round(graph_ms(separate_call, 4 * n_buf, 10, torch) * 1e3, 2)}
        temb16 = seeded_bf16(torch, dev, 2, 0, (4, Kg), 1.0)  # the same for a batch of four
        res["M4_with_silu"] = {"fused_us": round(graph_ms(fused_call, 4 * n_buf, 10, torch) * 1e3, 2),
                               "separate_us": round(graph_ms(separate_call, 4 * n_buf, 10, torch) * 1e3, 2)}
        gemv[f"w{bits_g}"] = res
        del bufs
    del gemv_w16

    # ---- secondary: the text stream of a joint block (M = 512) -----------------
    medium = {}
    for (Km, Nm) in (() if args.no_secondary else ((3072, 3072), (3072, 12288), (12288, 3072))):
        xm = torch.randn(512, Km, device=dev, generator=gen).to(torch.bfloat16)
        w = (torch.randn(Nm, Km, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        wqm, sm, bm = mflux_amd.quantize(w, GS, BITS)
        del w
        ms = graph_ms(lambda: mflux_amd.quantized_matmul(xm, wqm, sm, bm, group_size=GS, bits=BITS), 10, 5, torch)
        medium[f"{Km}x{Nm}"] = {"us": round(ms * 1e3, 1), "tflops": round(2.0 * 512 * Km * Nm / ms / 1e9, 1)}

    # ---- secondary: what follows the linear, inside the GEMM against element-wise passes behind it ----
    #   single block: gelu_approx on proj_mlp's part of linear1 (columns from 9216 on), and
    #   residual + gate * linear2(.) (single_transformer_block.py:45-57);
    #   Z-Image: silu(w1 x) * w3 x at M = 4352, 3840 -> 2 x 10240, W8 (feed_forward.py:13).
    fused = {}
    if not args.no_secondary:
        from mflux_amd import nn as qnn

        def best_of(calls):
            for fn in calls.values():
                for _ in range(3):
                    fn()
            best = {key: float("inf") for key in calls}
            for _ in range(3):
                for key, fn in calls.items():
                    best[key] = min(best[key], event_ms(fn, 10, torch))
            return {key: round(ms * 1e3, 1) for key, ms in best.items()}

        (_, x1, wq1, s1, b1), (_, x2, wq2, s2, b2) = ops
        fused["linear1_gelu_from_9216"] = best_of({
            "fused_us": lambda: mflux_amd.quantized_matmul_epilogue(x1, wq1, s1, b1, epilogue="gelu", group_size=GS,
                                                                    bits=BITS, act_from=9216),
            "separate_us": lambda: torch.cat([(y := mflux_amd.quantized_matmul(x1, wq1, s1, b1, group_size=GS, bits=BITS))[:, :9216],
                                              mflux_amd.gelu_approx(y[:, 9216:])], dim=1),
        })
        gate = seeded_bf16(torch, dev, CONFIG, 30, (3072,), 1.0)
        res = seeded_bf16(torch, dev, CONFIG, 31, (M_TOKENS, 3072), 1.0)
        fused["linear2_gate_residual"] = best_of({
            "fused_us": lambda: mflux_amd.quantized_matmul_epilogue(x2, wq2, s2, b2, epilogue="gate_residual",
                                                                    group_size=GS, bits=BITS, gate=gate, residual=res),
            "separate_us": lambda: res + gate * mflux_amd.quantized_matmul(x2, wq2, s2, b2, group_size=GS, bits=BITS),
        })
        del gate, res
        xz = seeded_bf16(torch, dev, 4, 10, (4352, 3840), 1.0)
        halves = []
        for idx in (11, 21):
            lin = qnn.QuantizedLinear(3840, 10240, bias=False, group_size=GS, bits=8)
            lin.weight, lin.scales, lin.biases = mflux_amd.quantize(seeded_bf16(torch, dev, 4, idx, (10240, 3840), 0.02), GS, 8)
            halves.append(lin)
        stacked = qnn.stack_gate_up(*halves)
        fused["zimage_swiglu_3840_to_2x10240_w8"] = best_of({
            "fused_us": lambda: qnn.swiglu_linear(stacked, xz),
            "separate_us": lambda: mflux_amd.silu(halves[0](xz)) * halves[1](xz),
        })
        del xz, halves, stacked
        # the step in front of the modulated linears: LayerNorm(x) * (1 + scale) + shift over [4608, 3072]
        xn = seeded_bf16(torch, dev, CONFIG, 40, (M_TOKENS, 3072), 1.0)
        scn, shn = seeded_bf16(torch, dev, CONFIG, 41, (3072,), 0.3), seeded_bf16(torch, dev, CONFIG, 42, (3072,), 0.3)
        # (10 us kernels: back to back in a HIP graph, as the matvecs are timed)
        fused["layer_norm_modulate_4608x3072"] = {
            "fused_us": round(graph_ms(lambda: mflux_amd.layer_norm_modulate(xn, scn, shn), 16, 5, torch) * 1e3, 2),
            "separate_us": round(graph_ms(
                lambda: torch.nn.functional.layer_norm(xn, (3072,), eps=1e-6) * (1 + scn) + shn, 16, 5, torch) * 1e3, 2),
        }
        fused["layer_norm_modulate_4608x3072"]["frac_hbm"] = round(
            2 * 2 * M_TOKENS * 3072 / (fused["layer_norm_modulate_4608x3072"]["fused_us"] * 1e-6) / 1e9 / PEAK_HBM_GBS, 4)
        del xn, scn, shn

    configs = {} if args.no_secondary else baseline_configs(torch, mflux_amd, dev, quick=args.configs_quick)

    quant = {}
    for (name, K, N) in (() if args.no_secondary else LINEARS):
        ms = quant_ms[name]
        nbytes = quantize_bytes(N, K, BITS)
        gbs = nbytes / (ms * 1e-3) / 1e9
        quant[name] = {"us": round(ms * 1e3, 1), "GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4)}

    # the second half of the headline metric ("W8 GEMV GB/s at M=1") in the form of `roofline`: algorithmic
    # bytes of one 3072 -> 18432 call over its time in a chain of graph launches; traffic from the committed
    # FETCH_SIZE / WRITE_SIZE profile of the same kernel (62.7 MB read, 0.04 MB written)
    gemv_roofline = None
    if "w8" in gemv:
        m1 = gemv["w8"]["M1"]
        gemv_traffic, gemv_traffic_source = profiled_traffic("gemv")
        gemv_roofline = {"kernel": "qmv_oct_kernel<BF16,3,1>", "bound": "hbm", "achieved": m1["GB/s"],
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": m1["frac_hbm"], "traffic": gemv_traffic,
                         "traffic_source": gemv_traffic_source,
                         "avg_launch_us": m1["us"], "bytes_per_launch": m1["bytes"]}
    out = {
        "metric": "W4A16 qmatmul TFLOP/s @ FLUX single-block M=4608",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "flux1_single_block_1024px_m4608_w4_gs64: linear1 3072->21504 + linear2 15360->3072",
                   "M": M_TOKENS, "bits": BITS, "group_size": GS},
        "roofline": roofline,
        "per_shape": per_shape,
        "secondary": {"metric": "W8 GEMV GB/s (adaLN 3072->18432, cold weights)", "roofline": gemv_roofline,
                      "gemv_w8": gemv.get("w8", {}),
                      "gemv_w4": gemv.get("w4", {}), "quantize_w4": quant, "qmm_w4_m512": medium,
                      "qmm_w4_lora_r16": lora, "epilogues_fused_vs_separate": fused,
                      "library_bf16_gemm_same_operands": library, "qmm_w4_prepared_weights": prepared,
                      "configs": configs},
    }
    if not args.no_cpu_baseline:
        name, x, wq, s, b = ops[0]
        out["cpu_baseline"] = cpu_baseline(torch, x, wq, s, b, args.cpu_sample_rows)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
