"""What one MI355X sustains on the instructions the NCN kernels are made of.

    python -m ncn_cuda_amd.probe [--iters N]

Prints, for each instruction kind (in the operand forms that matter: sources in vector registers, a scalar-register
source, a DPP operand; two mixes shaped like one element-step of the forward and of the backward step code; one
instruction kind among FMAs), the time of a launch that issues nothing else, at 1, 2, 4 and 8 resident waves per SIMD and 1, 4 and 8
independent dependency chains per lane:

    cycles = launch time x 2.4 GHz / (wave instructions issued per SIMD)     (2.4 GHz: the GPU's peak engine clock)
    TFLOP/s = floating-point operations / launch time                         (FMA = 2)

The kernels (csrc/ncn_probe.hip, entry point ncn_probe_issue) are built like the rest of the library, without packed
FP32 instructions.  `fma_stream_tflops()` is the one figure bench.py quotes as `roofline.attainable_valu_TFLOPs`.
"""
import argparse
import ctypes

import torch

from . import _lib

MODES = ["v_fma_f32 (vector registers)", "v_add_f32", "v_mul_f32", "v_exp_f32", "v_rcp_f32", "exp2, +1, rcp",
         "v_add_f32 dpp quad_perm", "ds_swizzle + v_add_f32", "backward step mix", "forward step mix",
         "v_mfma_f32_16x16x4_f32", "4 v_fma_f32 + 1 independent mfma", "v_fmac_f32 with a scalar source",
         "1 scalar-source fmac : 3 v_fma_f32", "1 v_exp_f32 : 7 v_fma_f32", "1 dpp add : 1 v_fma_f32"]
PEAK_CLOCK_HZ = 2.4e9


def time_launch(mode, chains, waves, iters, reps=3, device=None):
    """Best of `reps` launches: (milliseconds, wave instructions per SIMD, floating-point operations of the launch)."""
    lib = _lib.load()
    dev = torch.device("cuda:0") if device is None else device
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    out = torch.empty(8 * cus * 256, dtype=torch.float32, device=dev)
    valu, flops = ctypes.c_int(0), ctypes.c_int(0)
    groups = lib.ncn_probe_issue_info(mode, ctypes.byref(valu), ctypes.byref(flops))
    if groups <= 0:
        raise ValueError(f"unknown probe mode {mode}")
    stream = torch.cuda.current_stream(dev).cuda_stream
    with torch.cuda.device(dev):
        _lib.check(lib.ncn_probe_issue(mode, chains, waves, iters, out.data_ptr(), stream), "ncn_probe_issue")
        best = None
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _lib.check(lib.ncn_probe_issue(mode, chains, waves, iters, out.data_ptr(), stream), "ncn_probe_issue")
            e1.record()
            torch.cuda.synchronize(dev)
            ms = e0.elapsed_time(e1)
            best = ms if best is None or ms < best else best
    per_lane_groups = iters * groups * chains
    wave_instr_per_simd = per_lane_groups * valu.value * waves          # one wave per SIMD and workgroup
    total_flops = per_lane_groups * flops.value * 64.0 * 4 * cus * waves
    return best, wave_instr_per_simd, total_flops


def fma_stream_tflops(iters=2048, device=None):
    """v_fma_f32 on vector registers, 8 chains per lane, 8 waves per SIMD: the float32 vector rate without packed
    instructions."""
    ms, _, flops = time_launch(0, 8, 8, iters, device=device)
    return flops / (ms * 1e-3) / 1e12


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=2048)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("the probe needs a GPU")
    props = torch.cuda.get_device_properties(0)
    print(f"device {props.name}, {props.multi_processor_count} CUs, library {_lib.load().ncn_version().decode()} "
          f"(build {_lib.load().ncn_build_id().decode()}); cycles at {PEAK_CLOCK_HZ / 1e9:.1f} GHz")
    print(f"{'instructions':34s} {'waves/SIMD':>10s} {'chains':>6s} {'ms':>8s} {'cycles/instr':>12s} {'TFLOP/s':>8s}")
    for mode, name in enumerate(MODES):
        for waves in (1, 2, 4, 8):
            for chains in (1, 4, 8):
                ms, instr, flops = time_launch(mode, chains, waves, args.iters)
                rate = f"{flops / (ms * 1e-3) / 1e12:8.2f}" if flops else f"{'-':>8s}"
                print(f"{name:34s} {waves:10d} {chains:6d} {ms:8.3f} {ms * 1e-3 * PEAK_CLOCK_HZ / instr:12.2f} {rate}",
                      flush=True)


if __name__ == "__main__":
    main()
