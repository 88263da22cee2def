#!/usr/bin/env python3
"""Benchmark of the BitLinear W1.58A8 forward path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one token at batch 1 through the decode projections of a BitNet-b1.58-2B stack: 30 passes of the
decoder-layer workload (hidden 2560, FFN 6912, 20 query / 5 KV heads: fused RMSNorm + int8 quantisation before
q/k/v and before gate/up, int8 quantisation before o and down, seven packed-ternary GEMVs with the scale
epilogue), each over the weights of its own layer (521 MB of packed weights per step, more than the last-level
cache holds, so no pass finds its weights cached), the hidden state carried from layer to layer.  Inputs and
weights are resident in HBM before the timed region: one untimed step comes first (first touch of every weight
page), then the warm-up steps, then the region of exactly K steps, which is run REPEATS times back to back; the
line reports the median region (every region's time is listed under config.region_ms).  A step is long enough
(about 0.5 ms) for the cost of starting and stopping a region to vanish, so a short run (--steps 20) and a long
one agree.  value = packed-weight bytes streamed per second over that region, by the host's clock around it;
config.us_per_layer is the same figure per decoder layer.

The timed region contains one kernel family only, the decode GEMV with the activation quantiser fused into
its prologue (four launches per layer: q+k+v, o, gate+up, down), so the roofline of the dominant kernel comes
straight from the HIP events around the timed region: achieved = packed-weight bytes per launch / average
launch duration.  The line also carries the GEMV alone on pre-quantised activations (graph replays over the
same 210 matrices), the prefill GEMM rate (M = 2048) at the two FFN shapes, and a CPU baseline (a C
restatement of the reference's dequantise-to-f32 BitLinear forward) timed on this host's cores for a bounded
sample.
"""
import argparse
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT / "bitnet-mlx.rs_amd" / "python"))
sys.path.insert(0, str(ROOT))

HIDDEN, FFN, Q_HEADS, KV_HEADS, HEAD_DIM, LAYERS = 2560, 6912, 20, 5, 128, 30
LAYER_BYTES = 17_367_040  # sum of n*k/4 over q,k,v,o,gate,up,down
HBM_PEAK_GBS = 8000.0
INT8_PEAK_TOPS = 5000.0


def build_stack(bh, torch, layers, max_tokens=1):
    dec = bh.DecoderProjections(layers, HIDDEN, FFN, Q_HEADS, KV_HEADS, HEAD_DIM, eps=1e-5, max_tokens=max_tokens)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    for l in range(layers):
        for p in range(7):
            n, k = dec.proj_shape(p)
            w = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
            dec.projection(l, p).update_weights(w)  # ternarised, packed and re-tiled on the GPU
            del w
    return dec, gen


def time_events(torch, fn):
    """Elapsed milliseconds of fn() measured with events on the stream the kernels are launched on."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop)


REPEATS = 7  # timed regions of --steps steps each; the median is reported
LAUNCHES_PER_LAYER = 4  # q+k+v | o | gate+up | down, each one gemv_fused16_kernel<MODE, NORM, NCHB, RBW> launch
# A step is one token at batch 1 through the decode projections of all 30 layers (30 passes of the decoder-layer
# workload, each over its own weights, the hidden state carried from layer to layer): 120 dependent launches, 521 MB
# of packed weights, about 0.5 ms.  Starting and stopping a timed region costs 20 to 90 us on the boxes measured
# (event records, the first launch into an idle queue, the wake-up of the waiting host thread); with a step this
# long that is under 1 % of a region of 20 steps, so the figure does not depend on --steps.
LAUNCHES_PER_STEP = LAUNCHES_PER_LAYER * LAYERS
STEP_BYTES = LAYER_BYTES * LAYERS
# HBM bytes per launch of that kernel from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (two runs of this
# script with --no-extras --calibration-copy), each scaled by what the same counter reads for the plain
# 256 MiB copy: FETCH_SIZE reads 0.5 KiB per KiB fetched (factor 2.0), WRITE_SIZE 1.0 (factor 1.0).
# Summary: profiles/decode_layer_b1_gemv_hbm_traffic.md
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = 4_685_621


def decode_roofline(event_ms, steps):
    launches = steps * LAUNCHES_PER_STEP
    total_bytes = steps * STEP_BYTES
    achieved = total_bytes / (event_ms * 1e-3) / 1e9
    return {
        "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH,
        "kernel": "gemv_fused16_kernel<MODE, NORM, NCHB, RBW> (decode GEMV, activation quantiser in the prologue)",
        "launches": launches, "avg_launch_us": round(event_ms * 1e3 / launches, 3),
        "bytes_per_launch": LAYER_BYTES // LAUNCHES_PER_LAYER,
        "how": "HIP events on the launch stream around the timed region, which holds only this kernel "
               "(4 launches per layer, 120 per step, back to back); algorithmic bytes = packed weights n*k/4",
    }


def gemv_only(bh, torch, dec, gen, reps):
    """The GEMV alone on pre-quantised int8 activations: one launch per projection over all 210 matrices,
    captured in a HIP graph so that host launch cost does not starve the GPU; HIP events around the replays."""
    a = {k: torch.randint(-127, 128, (1, k), generator=gen, device="cuda", dtype=torch.int8) for k in (HIDDEN, FFN)}
    a_scale = torch.ones((1,), device="cuda", dtype=torch.float32)
    outs = {n: torch.empty((1, n), device="cuda", dtype=torch.float32) for n in (HIDDEN, KV_HEADS * HEAD_DIM, FFN)}
    projs = [(dec.projection(l, p), dec.proj_shape(p)) for l in range(dec.layers) for p in range(7)]

    def launch_all():
        for bl, (n, k) in projs:
            bl.matmul_quantized(a[k], a_scale, out=outs[n])

    launch_all()
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            launch_all()
        graph.replay()
        torch.cuda.synchronize()
        ms = time_events(torch, lambda: [graph.replay() for _ in range(reps)])
    launches = reps * len(projs)
    total_bytes = reps * dec.weight_bytes()
    return {"kernel": "gemv_tiled_kernel<1, -1>", "launches": launches, "avg_launch_us": round(ms * 1e3 / launches, 3),
            "bytes_per_launch": round(total_bytes / launches), "gbs": round(total_bytes / (ms * 1e-3) / 1e9, 1)}


PREFILL_LOOPS, PREFILL_LAUNCHES = 7, 50  # the prefill GEMM is timed as the median of 7 loops of 50 back-to-back launches


def median_loop_ms(torch, fn, launches, loops):
    """Milliseconds per launch: the median over `loops` event-timed loops of `launches` back-to-back calls of fn."""
    times = sorted(time_events(torch, lambda: [fn() for _ in range(launches)]) / launches for _ in range(loops))
    return times[len(times) // 2], times


def prefill_rates(bh, torch, dec, gen, reps):
    """configs[3]: the M = 2048 prefill GEMM at the two FFN shapes, on the configuration's own operands: f32 rows ~ N(0,1)
    quantised per token by the library's quantiser (int8, a_scale, a_sum), ternary weights from N(0, 0.02)."""
    m = 2048
    res = {}
    launches, loops = max(reps, 1), (PREFILL_LOOPS if reps >= PREFILL_LAUNCHES else 3)
    for name, p in (("2048x2560x6912", 4), ("2048x6912x2560", 6)):
        n, k = dec.proj_shape(p)
        bl = dec.projection(0, p)
        x = torch.randn((m, k), generator=gen, device="cuda", dtype=torch.float32)
        a, a_scale, a_sum, _ = bh.quantize_activations_i8(x, want_sum=True)
        out = torch.empty((m, n), device="cuda", dtype=torch.float32)
        bl.matmul_quantized(a, a_scale, out=out, a_sum=a_sum)
        ms, all_ms = median_loop_ms(torch, lambda: bl.matmul_quantized(a, a_scale, out=out, a_sum=a_sum), launches, loops)
        tops = 2.0 * m * n * k / (ms * 1e-3) / 1e12
        res[name] = {"ms": round(ms, 4), "tops": round(tops, 1), "frac_int8_mfma_peak": round(tops / INT8_PEAK_TOPS, 4),
                     "timed": f"median of {loops} loops of {launches} launches, operands of configs[3] (quantised N(0,1) rows)",
                     "loops_ms": [round(t, 4) for t in all_ms]}
        # the whole BitLinear forward on f32 activations (absmax int8 quantiser + GEMM + scale epilogue), for reference
        bl.forward(x)
        fwd_ms, _ = median_loop_ms(torch, lambda: bl.forward(x), min(launches, 20), 3)
        res[name]["forward_f32_in_ms"] = round(fwd_ms, 4)
        # calibration only: the vendor library's int8 GEMM (torch._int_mm -> hipBLASLt) at the same shape, on weights
        # expanded to one int8 per value and without the scale epilogue (int32 output); not part of the measured path
        try:
            w8 = torch.randint(-1, 2, (n, k), generator=gen, device="cuda", dtype=torch.int8)
            torch._int_mm(a, w8.t())
            lib_ms, _ = median_loop_ms(torch, lambda: torch._int_mm(a, w8.t()), min(launches, 20), 3)
            res[name]["vendor_int8_gemm_ms"] = round(lib_ms, 4)
            res[name]["vendor_int8_gemm_tops"] = round(2.0 * m * n * k / (lib_ms * 1e-3) / 1e12, 1)
            del w8
        except Exception as exc:  # the calibration must never fail the benchmark
            res[name]["vendor_int8_gemm_ms"] = None
            res[name]["vendor_int8_gemm_note"] = repr(exc)[:120]
        del a, out, x
    # projections that share their input in one call: one quantiser pass, one GEMM launch for all of them
    x = torch.randn((m, HIDDEN), generator=gen, device="cuda", dtype=torch.float32)
    for name, projs in (("q_k_v_2048x3840x2560", (0, 1, 2)), ("gate_up_2048x13824x2560", (4, 5))):
        layers = [dec.projection(0, p) for p in projs]
        bh.forward_multi(layers, x)
        ms, _ = median_loop_ms(torch, lambda: bh.forward_multi(layers, x), min(launches, 20), 3)
        ops = 2.0 * m * HIDDEN * sum(dec.proj_shape(p)[0] for p in projs)
        res[name] = {"forward_f32_in_ms": round(ms, 4), "tops_incl_quantiser": round(ops / (ms * 1e-3) / 1e12, 1)}
    # what the matrix unit of this device sustains when it does nothing but v_mfma_i32_16x16x64_i8 from registers: the
    # practical ceiling under the published 5.0 POP/s (its clock under load and the operands' switching activity included)
    rand_tops, const_tops = bh.measure_mfma_i8_rate(True), bh.measure_mfma_i8_rate(False)
    res["mfma_loop_ceiling"] = {"tops_random_operands": round(rand_tops, 1), "tops_constant_operands": round(const_tops, 1),
                                "frac_int8_mfma_peak": round(rand_tops / INT8_PEAK_TOPS, 4)}
    for name in ("2048x2560x6912", "2048x6912x2560"):
        res[name]["frac_of_mfma_loop"] = round(res[name]["tops"] / rand_tops, 4)
    return res


def large_gemv_pair(bh, torch, gen, loops=5):
    """The decode GEMV where a launch is large enough to be bound by bandwidth rather than by launch latency: 32768 x 16384
    ternary weights, int8 activations already quantised, one token; on the 2-bit streaming layout (128 MiB per matrix)
    and on base-3 bytes (five weights per byte, 102 MiB: 20 % fewer bytes, every byte through a table in LDS).  Four
    matrices in rotation each, more than the last-level cache holds."""
    out = {}
    n, k = 32768, 16384
    layers = [bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), f"large{i}") for i in range(4)]  # 512 MiB > cache
    packed = torch.randint(0, 256, (n * k // 4,), generator=gen, device="cuda", dtype=torch.uint8)
    for bl in layers:
        bl.set_quantized_weights(packed, 0.02)
    a = torch.randint(-127, 128, (1, k), generator=gen, device="cuda", dtype=torch.int8)
    a_scale = torch.ones((1,), device="cuda", dtype=torch.float32)
    y = torch.empty((1, n), device="cuda", dtype=torch.float32)
    for bl in layers:
        bl.matmul_quantized(a, a_scale, out=y)
    # median of five event-timed regions of `loops` passes over the four matrices (the first region runs on cold clocks)
    regions = sorted(time_events(torch, lambda: [bl.matmul_quantized(a, a_scale, out=y) for _ in range(loops) for bl in layers])
                     / (4 * loops) for _ in range(5))
    ms = regions[2]
    out["gemv_32768x16384_m1"] = {"us": round(ms * 1e3, 2), "gbs_packed_weights": round(n * k / 4 / (ms * 1e-3) / 1e9, 1),
                                  "frac_hbm_peak": round(n * k / 4 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                  "best_region_frac_hbm_peak": round(n * k / 4 / (regions[0] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                  "timed": f"median of 5 regions of {4 * loops} launches over 4 x 128 MiB of distinct weights (the rate "
                                           "sags by a few per cent while the stream is sustained: every region is listed)",
                                  "regions_us": [round(r * 1e3, 2) for r in regions]}
    del layers, packed
    b3_bytes = bh.base3_packed_size(n * k)
    tiled3 = [bh.retile_base3(torch.randint(0, 243, (b3_bytes,), generator=gen, device="cuda", dtype=torch.uint8), n, k)
              for _ in range(4)]
    for t3 in tiled3:
        bh.gemv_base3(t3, a.view(-1), n, want_acc=False, w_scale=a_scale, out=y.view(-1))
    ms3 = sorted(time_events(torch, lambda: [bh.gemv_base3(t3, a.view(-1), n, want_acc=False, w_scale=a_scale, out=y.view(-1))
                                             for _ in range(loops) for t3 in tiled3]) / (4 * loops) for _ in range(5))[2]
    out["gemv_base3_32768x16384_m1"] = {
        "us": round(ms3 * 1e3, 2), "bytes_per_launch": b3_bytes,
        "gbs_base3_bytes": round(b3_bytes / (ms3 * 1e-3) / 1e9, 1),
        "frac_hbm_peak": round(b3_bytes / (ms3 * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "speed_vs_2bit_gemv": round(ms / ms3, 3),
        "note": "the decode GEMV consuming Base3PackedPacker bytes (1.6 bits per weight) directly; bound by the LDS table "
                "look-ups that take a byte apart, not by memory"}
    return out


def stack_latency(bh, torch, dec, gen, reps=20):
    """configs[4]: per-token decode latency through all 30 layers' projections, batch 1 and batch 8, and
    configs[2]: the gate / down projections at M in {1, 4, 16, 64} tokens (activations with 1 % x20 outliers)."""
    out = {}
    big = bh.DecoderProjections(dec.layers, HIDDEN, FFN, Q_HEADS, KV_HEADS, HEAD_DIM, eps=1e-5, max_tokens=8)
    for l in range(dec.layers):
        for p in range(7):
            packed, scale = dec.projection(l, p).get_quantized_weights()
            big.projection(l, p).set_quantized_weights(packed.cuda(), scale)
    for m in (1, 8):
        x = torch.randn((m, HIDDEN), generator=gen, device="cuda", dtype=torch.float32)
        y = torch.empty_like(x)
        big.decode(x, out=y)
        eager_ms = time_events(torch, lambda: [big.decode(x, out=y) for _ in range(reps)]) / reps
        recorded = big.record(x, out=y)
        recorded.replay()
        ms = sorted(time_events(torch, lambda: [recorded.replay() for _ in range(reps)]) / reps for _ in range(3))[1]
        out[f"stack30_batch{m}"] = {"us_per_token_step": round(ms * 1e3, 1),
                                    "gbs_packed_weights": round(dec.weight_bytes() / (ms * 1e-3) / 1e9, 1),
                                    "eager_launches_us_per_token_step": round(eager_ms * 1e3, 1),
                                    "timed": "the recorded step replayed (HIP graph); eager = launches enqueued one by one"}
        del recorded
    del big
    out.update(large_gemv_pair(bh, torch, gen))
    for name, p in (("gate_2560x6912", 4), ("down_6912x2560", 6)):
        n, k = dec.proj_shape(p)
        bls = rotating_layers(bh, torch, dec, gen, p)  # 60 x 4.4 MB = 265 MB: more than the last-level cache holds
        bl = bls[0]
        for m in (1, 4, 16, 64):
            x = torch.randn((m, k), generator=gen, device="cuda", dtype=torch.float32)
            mask = torch.rand((m, k), generator=gen, device="cuda") < 0.01
            x = torch.where(mask, x * 20.0, x).contiguous()
            y = torch.empty((m, n), device="cuda", dtype=torch.float32)
            ws = torch.empty((max(bl.workspace_size(m), 16),), device="cuda", dtype=torch.uint8)
            ms, how = time_forward_graph(torch, bls, x, y, ws)
            out[f"{name}_m{m}"] = {"us": round(ms * 1e3, 2), "gbs_packed_weights": round(n * k / 4 / (ms * 1e-3) / 1e9, 1),
                                   "timed": how}
    out.update(short_prompt_forward(bh, torch, dec, gen))
    return out


_ROTATING = {}


def rotating_layers(bh, torch, dec, gen, proj):
    """Sixty layers of one projection's shape, each with its own weights (265 MB of packed tiles at 6912 x 2560: the
    256 MB last-level cache cannot hold them, so every pass fetches from HBM).  Gate and up have the same shape and serve
    each other; for down the stack's thirty are joined by thirty more with random ternary codes."""
    if proj in _ROTATING:
        return _ROTATING[proj]
    layers = [dec.projection(layer, proj) for layer in range(dec.layers)]
    if proj in (4, 5):
        layers += [dec.projection(layer, 9 - proj) for layer in range(dec.layers)]
    else:
        n, k = dec.proj_shape(proj)
        for i in range(dec.layers):
            bl = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), f"rotating{proj}_{i}")
            codes = torch.randint(0, 3, (n * k,), generator=gen, device="cuda", dtype=torch.uint8).view(-1, 4)
            packed = (codes[:, 0] | (codes[:, 1] << 2) | (codes[:, 2] << 4) | (codes[:, 3] << 6)).contiguous()
            bl.set_quantized_weights(packed, 0.02)
            layers.append(bl)
    _ROTATING[proj] = layers
    return layers


def short_prompt_forward(bh, torch, dec, gen):
    """Short prompts on the long-k projection (6912 -> 2560 at 128 and 256 tokens): forward (quantiser + GEMM) with the
    workspace forward asks for, which lets the GEMM split k across workgroups, and with one that holds the quantised
    activations only (no split)."""
    out = {}
    n, k = dec.proj_shape(6)
    bls = rotating_layers(bh, torch, dec, gen, 6)
    for m in (128, 256):
        x = torch.randn((m, k), generator=gen, device="cuda", dtype=torch.float32)
        y = torch.empty((m, n), device="cuda", dtype=torch.float32)
        quant_only = (m * k + 255) // 256 * 256 + 2 * ((4 * m + 255) // 256 * 256) + 256
        entry = {}
        for label, size in (("us", bls[0].workspace_size(m)), ("us_without_k_split", quant_only)):
            ws = torch.empty((size,), device="cuda", dtype=torch.uint8)
            ms, how = time_forward_graph(torch, bls, x, y, ws)
            entry[label] = round(ms * 1e3, 2)
        entry["tops_incl_quantiser"] = round(2.0 * m * n * k / (entry["us"] * 1e-6) / 1e12, 1)
        entry["timed"] = how
        out[f"down_6912x2560_m{m}_forward"] = entry
    return out


def launch_floor(bh, torch, step_us):
    """What a chain of 120 dependent launches costs on this device when the kernels do nothing, and when they only read the
    bytes the launches of a token step read (q+k+v, o, gate+up, down of 30 layers: the same 521 MB, distinct memory every
    launch): recorded as HIP graphs and replayed like the measured step, in this process.  The measured step cannot go
    below the second figure; the gap between the two is what reading the bytes adds to a launch."""
    per_launch = [(2560 * 2560 + 2 * 640 * 2560) // 4, 2560 * 2560 // 4, 2 * 6912 * 2560 // 4, 6912 * 2560 // 4]
    assert sum(per_launch) == LAYER_BYTES
    buf = torch.randint(0, 256, (STEP_BYTES,), device="cuda", dtype=torch.uint8)
    empty = sorted(bh.measure_launch_chain(LAUNCHES_PER_STEP, replays=20) for _ in range(5))[2]
    reads = sorted(bh.measure_launch_chain(LAUNCHES_PER_STEP, replays=20, buf=buf, bytes_per_launch=per_launch) for _ in range(5))[2]
    one = sorted(bh.measure_launch_chain(1, replays=20, buf=buf, bytes_per_launch=[STEP_BYTES]) for _ in range(5))[2]
    del buf
    # the alternative to a kernel boundary: workgroups that stay resident and hand the vector on through memory inside one
    # launch (bitnet_hip_measure_hop), at the three widths a layer hands over (v: 640, hidden state: 2560, gate / up: 6912)
    hop = {}
    for values in (640, 2560, 6912):
        for two_level in (False, True):
            us, intact = bh.measure_hop(values, hops=200, two_level=two_level)
            hop[f"{'two_level' if two_level else 'flat'}_{values}_values_us"] = round(us, 2) if intact else None
    return {"launches": LAUNCHES_PER_STEP, "bytes": STEP_BYTES, "in_launch_hand_over": hop,
            "empty_kernels_us_per_step": round(empty, 1), "empty_kernel_us_per_launch": round(empty / LAUNCHES_PER_STEP, 3),
            "read_only_kernels_us_per_step": round(reads, 1), "read_only_kernel_us_per_launch": round(reads / LAUNCHES_PER_STEP, 3),
            "read_only_frac_hbm_peak": round(STEP_BYTES / (reads * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "one_launch_reading_all_bytes_us": round(one, 1),
            "one_launch_frac_hbm_peak": round(STEP_BYTES / (one * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "measured_step_us": round(step_us, 1), "measured_over_read_only_floor": round(step_us / reads, 3),
            "how": "bitnet_hip_measure_launch_chain: a recorded chain of 120 dependent launches (kernels that do nothing / "
                   "kernels that only read the step's packed-weight bytes, 3.7 + 1.6 + 8.8 + 4.4 MB per layer), median of 5 "
                   "measurements of 20 replays each"}


def sequential_order_decode(bh, torch, dec, gen, reps=20):
    """The headline workload with the reference's literal RMSNorm summation order (one running f32 sum,
    inference_integration.rs:476) instead of the build's declared block order: same stack, same steps."""
    seq = bh.DecoderProjections(dec.layers, HIDDEN, FFN, Q_HEADS, KV_HEADS, HEAD_DIM, eps=1e-5, max_tokens=1,
                                sum_order=bh.SUM_SEQUENTIAL)
    for l in range(dec.layers):
        for p in range(7):
            packed, scale = dec.projection(l, p).get_quantized_weights()
            seq.projection(l, p).set_quantized_weights(packed.cuda(), scale)
    x = torch.randn((1, HIDDEN), generator=gen, device="cuda", dtype=torch.float32)
    y = torch.empty_like(x)
    seq.decode(x, out=y)
    times = sorted(time_events(torch, lambda: [seq.decode(x, out=y) for _ in range(reps)]) / reps for _ in range(5))
    ms = times[len(times) // 2]
    return {"us_per_layer_step": round(ms * 1e3 / dec.layers, 2), "gbs_packed_weights": round(dec.weight_bytes() / (ms * 1e-3) / 1e9, 1),
            "timed": f"median of 5 loops of {reps} 30-layer token steps"}


def eager_decode(torch, dec, x, reps=20):
    """The headline step with its 120 launches enqueued one by one by the host, and what that enqueue costs the host:
    where the host needs longer per launch than the GPU, the loop runs at the host's pace."""
    dec.decode(x, out=x)
    torch.cuda.synchronize()
    host = []
    for _ in range(9):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.decode(x, out=x)
        host.append(time.perf_counter() - t0)
    host_us = sorted(host)[len(host) // 2] * 1e6
    times = sorted(time_events(torch, lambda: [dec.decode(x, out=x) for _ in range(reps)]) / reps for _ in range(5))
    ms = times[len(times) // 2]
    return {"us_per_token_step": round(ms * 1e3, 1), "gbs_packed_weights": round(dec.weight_bytes() / (ms * 1e-3) / 1e9, 1),
            "host_enqueue_us_per_step": round(host_us, 1), "host_enqueue_us_per_launch": round(host_us / LAUNCHES_PER_STEP, 2),
            "timed": f"median of 5 loops of {reps} steps; enqueue = host time of one decode call into an idle queue"}


def time_forward_graph(torch, bls, x, y, ws, replays=10):
    """Device time of one BitLinear.forward (quantiser + GEMV launches): one forward per layer of `bls` captured
    into a HIP graph and replayed, so that the host's per-call cost (about 10 us through ctypes) is not what is
    measured.  Every replay is checked against the eager result; if capture is not possible the eager loop is
    timed instead."""
    calls = len(bls)
    for bl in bls:
        bl.forward(x, out=y, workspace=ws)
    torch.cuda.synchronize()
    want = y.clone()
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            bls[-1].forward(x, out=y, workspace=ws)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for bl in bls:
                bl.forward(x, out=y, workspace=ws)

        def checked_replay():
            y.zero_()
            graph.replay()
            torch.cuda.synchronize()
            if not torch.equal(y, want):
                raise RuntimeError("graph replay differs from the eager result")

        checked_replay()
        checked_replay()
        best = min(time_events(torch, graph.replay) for _ in range(replays))
        checked_replay()
        return best / calls, f"hip graph of {calls} forwards (each over its own weights), best of {replays} replays"
    except Exception as exc:  # capture unsupported: keep the measurement, say how it was made
        torch.cuda.synchronize()
        ms = time_events(torch, lambda: [bl.forward(x, out=y, workspace=ws) for bl in bls]) / calls
        return ms, f"eager loop of {calls} calls (graph capture failed: {type(exc).__name__})"


def cpu_baseline(torch, dec, budget_s=8.0):
    """The reference's CPU BitLinear on the host cores, one layer's seven projections at batch 1, three restatements:
    ref_f32  what BitLinear::forward executes per call: materialise q*scale as f32 [N,K], then an f32 GEMV
             (bitnet-quant/src/bitlinear/forward.rs:153-258); the headline figure of this object, all cores
    ref_simd the reference's ternary SIMD GEMV semantics: i8 weights widened to f32, FMA with f32 activations
             (bitnet-quant/src/simd/matrix.rs:287-368,471-490)
    oracle_i8 the int8 x ternary int32 path the GPU kernels reproduce (the oracle's BitLinear forward)
    each on all cores and on one thread, a bounded sample each."""
    import numpy as np

    from oracle import oracle as orc

    cores = orc.cpu_threads()
    mats = []
    for p in range(7):
        n, k = dec.proj_shape(p)
        packed, scale = dec.projection(0, p).get_quantized_weights()
        q = orc.unpack_2bit(packed.numpy(), n * k).reshape(n, k)
        mats.append((q, np.float32(scale), np.empty(n * k, dtype=np.float32), np.empty((1, n), dtype=np.float32), packed.numpy()))
    rng = np.random.default_rng(0)
    x = {k: rng.standard_normal((1, k), dtype=np.float32) for k in (HIDDEN, FFN)}

    def ref_f32():
        for q, s, wf, out, _ in mats:
            orc.cpu_ref_f32_forward(x[q.shape[1]], q, s, wf, out)

    def ref_simd():
        for q, s, _, out, _ in mats:
            orc.cpu_ref_simd_gemv(q, x[q.shape[1]], out, s)

    def oracle_i8():
        for q, s, _, _, packed in mats:
            orc.bitlinear_forward(x[q.shape[1]], packed, q.shape[0], s)

    def sample(fn, threads, budget):
        orc.cpu_set_threads(threads)
        fn()
        t0 = time.perf_counter()
        reps = 0
        while True:
            fn()
            reps += 1
            if time.perf_counter() - t0 > budget or reps >= 200:
                break
        dt = (time.perf_counter() - t0) / reps
        return {"gbs": round(LAYER_BYTES / dt / 1e9, 3), "ms_per_layer": round(dt * 1e3, 3), "threads": threads, "passes": reps}

    main_leg = sample(ref_f32, cores, budget_s)
    variants = {"ref_f32_1_thread": sample(ref_f32, 1, 3.0),
                "ref_simd_all_cores": sample(ref_simd, cores, 3.0), "ref_simd_1_thread": sample(ref_simd, 1, 3.0),
                "oracle_i8_all_cores": sample(oracle_i8, cores, 3.0), "oracle_i8_1_thread": sample(oracle_i8, 1, 3.0)}
    orc.cpu_set_threads(cores)
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            model = next((line.split(":", 1)[1].strip() for line in f if line.startswith("model name")), model)
    except OSError:
        pass
    return {
        "value": main_leg["gbs"], "unit": "GB/s", "cores": cores, "kind": "port", "cpu_model": model,
        "sample": f"{main_leg['passes']} passes over one layer's 7 projections at batch 1 (dequantise to f32 + f32 GEMV per call, "
                  f"{orc.cpu_isa()}), {main_leg['ms_per_layer']:.2f} ms per layer = {main_leg['ms_per_layer'] * LAYERS:.1f} ms per "
                  f"30-layer step of the GPU figure",
        "ms_per_layer": main_leg["ms_per_layer"], "ms_per_step": round(main_leg["ms_per_layer"] * LAYERS, 2), "variants": variants,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip roofline / prefill / CPU legs (profiling runs)")
    ap.add_argument("--eager", action="store_true",
                    help="time the token step as 120 launches enqueued one by one from the host instead of replaying the "
                         "recorded step (the eager loop is bound by the host's launch rate on most boxes)")
    ap.add_argument("--only-prefill", type=int, default=0, metavar="REPS",
                    help="run only the two M=2048 prefill GEMMs REPS times each and print their rates (profiling runs)")
    ap.add_argument("--only-batch8", type=int, default=0, metavar="STEPS",
                    help="run only STEPS token steps of the 30-layer stack at batch 8 (profiling runs)")
    ap.add_argument("--only-large-gemv", type=int, default=0, metavar="LOOPS",
                    help="run only the 32768 x 16384 one-token GEMV, on 2-bit tiles and on base-3 bytes, LOOPS times over four "
                         "matrices each (profiling runs)")
    ap.add_argument("--only-short-prompt", action="store_true",
                    help="run only forward at 128 and 256 tokens on the 6912 -> 2560 projection, with and without the k split "
                         "(profiling runs)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a kernel of known traffic, to scale rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the one-GPU BitLinear path; --gpus must be 1 (nothing here uses a second GPU)",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import bitnet_hip as bh

    bh.init(0)
    if args.only_large_gemv > 0:
        gen = torch.Generator(device="cuda")
        gen.manual_seed(0)
        print(json.dumps(large_gemv_pair(bh, torch, gen, loops=args.only_large_gemv)))
        return
    dec, gen = build_stack(bh, torch, LAYERS)
    if args.only_prefill > 0:
        print(json.dumps({"prefill": prefill_rates(bh, torch, dec, gen, reps=args.only_prefill)}))
        return
    if args.only_short_prompt:
        print(json.dumps(short_prompt_forward(bh, torch, dec, gen)))
        return
    if args.only_batch8 > 0:
        big = bh.DecoderProjections(LAYERS, HIDDEN, FFN, Q_HEADS, KV_HEADS, HEAD_DIM, eps=1e-5, max_tokens=8)
        for l in range(LAYERS):
            for p in range(7):
                packed, scale = dec.projection(l, p).get_quantized_weights()
                big.projection(l, p).set_quantized_weights(packed.cuda(), scale)
        x8 = torch.randn((8, HIDDEN), generator=gen, device="cuda", dtype=torch.float32)
        y8 = torch.empty_like(x8)
        recorded8 = big.record(x8, out=y8)
        recorded8.replay()
        ms = time_events(torch, lambda: [recorded8.replay() for _ in range(args.only_batch8)]) / args.only_batch8
        print(json.dumps({"stack30_batch8": {"us_per_token_step": round(ms * 1e3, 1), "steps": args.only_batch8}}))
        return
    x = torch.randn((1, HIDDEN), generator=gen, device="cuda", dtype=torch.float32)

    # The step is recorded once (bitnet_hip_decoder_graph_create: the 120 launches of decode() as a HIP graph) and
    # replayed: the same kernels in the same order, enqueued by one host call.
    recorded = None if args.eager else dec.record(x, out=x)

    def run_steps(count):
        """`count` token steps, each one call of the boundary: the seven projections of layers 0..29 in turn, the hidden
        state carried along (four launches per layer)."""
        for _ in range(count):
            if recorded is None:
                dec.decode(x, out=x)
            else:
                recorded.replay()

    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    run_steps(1)  # residency: every layer's weights touched once, untimed
    run_steps(args.warmup)
    torch.cuda.synchronize()
    regions = []  # (host seconds, event milliseconds) of each region of exactly args.steps steps
    for _ in range(REPEATS):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record()
        run_steps(args.steps)
        stop.record()
        torch.cuda.synchronize()
        regions.append((time.perf_counter() - t0, start.elapsed_time(stop)))
    regions_sorted = sorted(regions)
    elapsed, event_ms = regions_sorted[len(regions_sorted) // 2]  # the median region by host time

    value = args.steps * STEP_BYTES / elapsed / 1e9
    line = {
        "metric": "BitLinear decode GB/s (% HBM peak) + prefill int8 TOPS (% MFMA peak)",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed * 1e3 / args.steps, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "i8", "data": "synthetic",
        "config": {"workload": "configs[1]: one decoder layer's 7 decode projections at batch 1 "
                               "(hidden 2560, ffn 6912, 20q/5kv heads), passed 30 times per step over the 30 distinct "
                               "weight sets of a BitNet-2B stack (= one token step of configs[4] at batch 1); "
                               "a step = 30 layers = 120 dependent kernel launches, one host call"
                               + (" (launches enqueued one by one)" if args.eager else
                                  " (bitnet_hip_decoder_graph_launch: the recorded step replayed)"),
                   "enqueue": "eager launches" if args.eager else "recorded step (HIP graph)",
                   "layers_per_step": LAYERS, "bytes_per_step": STEP_BYTES, "bytes_per_layer": LAYER_BYTES,
                   "us_per_layer": round(elapsed * 1e6 / args.steps / LAYERS, 3),
                   "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
                   "event_ms_per_step": round(event_ms / args.steps, 5), "repeats": REPEATS, "reported": "median region",
                   "region_ms": [round(r[0] * 1e3, 4) for r in regions], "sum_order": "block256 (the build's declared order)",
                   "device": bh.device_info()},
    }
    line["roofline"] = decode_roofline(event_ms, args.steps)
    if not args.no_extras:
        # Both halves of the metric and the floors they are judged against live under "roofline": the decode GEMV chain
        # above, the prefill GEMM at the two shapes of configs[3], the decode GEMV where a launch is large enough to be
        # bound by bandwidth, and the cost of 120 dependent launches on this device.
        line["roofline"]["launch_floor"] = launch_floor(bh, torch, event_ms * 1e3 / args.steps)
        line["gemv_only"] = gemv_only(bh, torch, dec, gen, reps=5)
        line["prefill"] = prefill_rates(bh, torch, dec, gen, reps=PREFILL_LAUNCHES)
        line["roofline"]["prefill"] = {
            name: {"us": round(line["prefill"][name]["ms"] * 1e3, 2), "tops": line["prefill"][name]["tops"],
                   "frac": line["prefill"][name]["frac_int8_mfma_peak"]}
            for name in ("2048x2560x6912", "2048x6912x2560")}
        line["roofline"]["prefill"].update({
            "bound": "mfma", "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "ops_per_launch": 2 * 2048 * 2560 * 6912,
            "mfma_loop_ceiling_tops": line["prefill"]["mfma_loop_ceiling"]["tops_random_operands"],
            "how": line["prefill"]["2048x2560x6912"]["timed"]})
        line["other_configs"] = stack_latency(bh, torch, dec, gen)
        large = line["other_configs"]["gemv_32768x16384_m1"]
        line["roofline"]["large_gemv_frac"] = large["frac_hbm_peak"]
        line["roofline"]["large_gemv"] = {"shape": "32768x16384, one token", "us": large["us"], "gbs": large["gbs_packed_weights"],
                                          "frac": large["frac_hbm_peak"], "bytes_per_launch": 32768 * 16384 // 4}
        line["other_configs"]["decode_layer_b1_sum_order_sequential"] = sequential_order_decode(bh, torch, dec, gen)
        line["other_configs"]["decode_b1_eager_launches"] = eager_decode(torch, dec, x)
        if not args.no_cpu_baseline:
            line["cpu_baseline"] = cpu_baseline(torch, dec)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
