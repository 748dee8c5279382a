#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

A "step" is one pass of the hot path over one batch of synthetic input that is already resident in HBM.
Without --workload the five headline configurations run one after the other and the ONE JSON line carries config 2
as its headline fields (--steps / --warmup apply to it) and all five under "configs", each with its whole-step
throughput, the dominant kernel's roofline fraction and its CPU baseline.
Workloads (the headline configurations):
    bfp_qdq      config 2 (headline): block-FP quantize-dequantize, bf16 [8,2048,4096], width 8, exp 8, block [1,16]
    mxint_qdq    config 1: MXINT8 quantize-dequantize, fp32 [4096,4096], block 32
    mxint_linear config 3: MXINT8 Linear forward, 4096x4096x4096, fp32 in/out
    mxfp_linear  config 4: MXFP4(e2m1) weights x MXFP8(e4m3) activations Linear, M=8192 K=8192 N=28672
    decoder_layer config 5: Llama-style decoder layer, every nn.Linear -> LinearMXInt, batch 8 x seq 2048, bf16
Secondary workloads (other rows of the path, same JSON; --dtype bf16|f32|f16 where it applies):
    integer_qdq, minifloat_denorm_qdq, minifloat_ieee_qdq, minifloat_mx_qdq, mxfp_qdq   on [8,2048,4096]
    attn_prob    score -> probability chain of the MX-quantized attention on [4,32,2048,2048]
    decode_linear  LinearMXInt 8192 -> 28672 for 16 tokens (weight-streaming kernel); decode_linear_packed: the same
                   with the weight streamed as int8 codes + scale bytes; decode_linear_mxfp4: LinearMXFP with e2m1
                   weights on the block-scaled MFMA
    bmm_scores   the score product q k^T of an attention block on the batched matrix-core kernel (bound by writing
                 the scores)
    copy         calibration copy
Prints ONE JSON line.  `value` is algorithmic GB/s (Q-DQ) or TFLOP/s (Linear) over the whole timed region;
`roofline` is for the dominant kernel, timed with HIP events on the launch stream; `cpu_baseline` is the CPU
oracle timed on this box's host cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "fp8": 5000.0}


def make_bfp_input(torch, seed=1):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(8, 2048, 4096, generator=g, dtype=torch.float32)
    idx = torch.randperm(4096, generator=g)[:4]  # 0.1 % of the channels carry outliers
    x[..., idx] *= 50
    return x.to(torch.bfloat16)


def make_mxint_input(torch, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(4096, 4096, generator=g, dtype=torch.float32)


class Workload:
    name = ""
    # Defaults of --steps / --warmup.  The timed region has to last tens of milliseconds for the clocks and the memory
    # system to reach their steady state: 200 steps of a 45 us kernel (9 ms) read 5.7-5.9 TB/s where 1000 steps after
    # 300 warm-up steps read 6.5 TB/s.  Workloads with long steps override these.
    default_steps = 2000
    default_warmup = 300
    metric = ""
    unit = ""
    dtype = ""
    bound = "hbm"
    kernel = ""

    def setup(self, torch, dev, n_buffers):
        raise NotImplementedError

    def step(self, i):
        raise NotImplementedError

    def work_per_step(self) -> float:
        """algorithmic bytes (hbm) or flops (mfma) per step"""
        raise NotImplementedError

    def cpu_baseline(self, torch, budget_s):
        return None


class BfpQdq(Workload):
    name = "bfp_qdq"
    metric = "block-FP quantize-dequantize throughput (algorithmic bytes: 2 B read + 2 B written per element)"
    unit = "GB/s"
    dtype = "bf16"
    kernel = "bfp_run_kernel"
    config = {"workload": "block_fp_quantizer bf16 [8,2048,4096] width=8 exponent_width=8 block=[1,16], "
                          "N(0,1) with 4 of 4096 channels x50, seed 1"}
    kw = dict(width=8, exponent_width=8, exponent_bias=None, block_size=[1, 16], skip_first_dim=True)

    def setup(self, torch, dev, n_buffers):
        import mase_amd.quantizers as Q

        self.Q = Q
        self.host = make_bfp_input(torch)
        # distinct buffers so that the 256 MB last-level cache cannot serve the reads of the next step
        self.bufs = [self.host.to(dev) if i == 0 else None for i in range(n_buffers)]
        for i in range(1, n_buffers):
            self.bufs[i] = self.bufs[0].roll(i, dims=1).contiguous()
        self.out = None

    def step(self, i):
        self.out = self.Q.block_fp_quantizer(self.bufs[i % len(self.bufs)], **self.kw)

    def work_per_step(self):
        return float(self.host.numel() * 4)

    def cpu_baseline(self, torch, budget_s):
        import oracle as O

        x = self.host
        O.block_fp_quantizer(x[:1].clone(), **self.kw)  # warm
        t0 = time.perf_counter()
        n = 0
        while True:
            O.block_fp_quantizer(x.clone(), **self.kw)
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 20:
                break
        dt = (time.perf_counter() - t0) / n
        return {"value": self.work_per_step() / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                "kind": "port", "sample": f"{n} full passes of the same [8,2048,4096] bf16 tensor, {dt*1e3:.0f} ms each"}


class MxintQdq(Workload):
    name = "mxint_qdq"
    metric = "MXINT8 quantize-dequantize throughput (algorithmic bytes: 4 B read + 4 B written per element)"
    unit = "GB/s"
    dtype = "f32"
    kernel = "mxint_qdq_vec_kernel"
    config = {"workload": "mxint_quantizer fp32 [4096,4096] block_size=32 element_bits=8 scale_bits=8, N(0,1) seed 0"}

    def setup(self, torch, dev, n_buffers):
        import mase_amd.quantizers as Q

        self.Q = Q
        self.host = make_mxint_input(torch)
        n_buffers = max(n_buffers, 8)  # 64 MB each: rotate over more of them
        self.bufs = [self.host.to(dev).roll(i, dims=0).contiguous() for i in range(n_buffers)]

    def step(self, i):
        self.out = self.Q.mxint_quantizer(self.bufs[i % len(self.bufs)], 32, 8)

    def work_per_step(self):
        return float(self.host.numel() * 8)

    def cpu_baseline(self, torch, budget_s):
        import oracle as O

        x = self.host
        O.mxint_quantizer(x[:64], 32, 8)
        t0 = time.perf_counter()
        n = 0
        while True:
            O.mxint_quantizer(x, 32, 8)
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 20:
                break
        dt = (time.perf_counter() - t0) / n
        return {"value": self.work_per_step() / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                "kind": "port", "sample": f"{n} full passes of the same [4096,4096] fp32 tensor, {dt*1e3:.0f} ms each"}


class CopyBytes(Workload):
    """calibration: a plain streaming copy of the same size as the default workload (128 MiB in, 128 MiB out)"""
    name = "copy"
    metric = "streaming copy throughput (bytes read + bytes written)"
    unit = "GB/s"
    dtype = "u8"
    kernel = "copy_bytes_kernel"
    config = {"workload": "plain streaming copy of 134217728 bytes (calibration: achievable HBM ceiling, counter scale)"}
    nbytes = 134217728

    def setup(self, torch, dev, n_buffers):
        import bench_support
        from mase_amd import _lib

        self.lib = bench_support.load()
        self._lib = _lib
        self.bufs = [torch.randint(0, 255, (self.nbytes,), dtype=torch.uint8, device=dev) for _ in range(max(n_buffers, 4))]
        self.outs = [torch.empty(self.nbytes, dtype=torch.uint8, device=dev) for _ in range(2)]

    def step(self, i):
        src, dst = self.bufs[i % len(self.bufs)], self.outs[i % 2]
        self._lib.check(self.lib.bench_copy_bytes(src.data_ptr(), dst.data_ptr(), self.nbytes, self._lib.stream_ptr(src)), "copy")

    def work_per_step(self):
        return 2.0 * self.nbytes


class _MfmaIssueRate(Workload):
    """calibration: v_mfma_f32_32x32x16_bf16 on register operands with nothing else running, two wavefronts per SIMD on
    every CU.  The rate depends on the operand values (the part holds the instruction back when operand bits vary), so
    it is measured for zeros and for uniform values; the second is the ceiling of a bf16 GEMM on real data."""
    default_steps, default_warmup = 40, 10
    unit = "TFLOP/s"
    dtype = "bf16"
    bound = "mfma"
    kernel = "probe_mfma_bf16_kernel"
    operands = 0
    iters = 4096      # x 8 instructions per wavefront
    work_groups = 256
    entry = "bench_probe_mfma_bf16"
    instruction = "v_mfma_f32_32x32x16_bf16"
    flop_per_instruction = 2.0 * 32 * 32 * 16
    nominal_cycles = 32
    instructions_per_iter = 8

    def setup(self, torch, dev, n_buffers):
        import bench_support
        from mase_amd import _lib

        self.lib = bench_support.load()
        self._lib = _lib
        self.out = torch.empty(self.work_groups * 512 + 4, dtype=torch.float32, device=dev)
        self.metric = f"matrix-core issue rate of {self.instruction} on register operands (no memory traffic)"
        self.config = {"workload": f"{self.work_groups} work-groups x 8 wavefronts x {self.instructions_per_iter * self.iters} instructions, operands: "
                                   + ("zeros" if self.operands == 0 else self.random_kind)}
        self.fn = getattr(self.lib, self.entry)

    random_kind = "uniform in [-2, 2)"

    def step(self, i):
        self._lib.check(self.fn(self.out.data_ptr(), self.out.numel() * 4, self.work_groups, 2, self.iters,
                                self.operands, self._lib.stream_ptr(self.out)), "probe")

    def work_per_step(self):
        return float(self.work_groups * 8 * self.instructions_per_iter * self.iters) * self.flop_per_instruction

    def extra(self, torch):
        """shader clock during the last launch, from the kernel's own two counters (first wavefront's loop)"""
        cyc, ticks = self.out[-4:].view(torch.int64).tolist()
        rate_khz = int(self.lib.bench_constant_rate_counter_khz())
        secs = ticks / (rate_khz * 1e3)
        return {"shader_clock_ghz_in_loop": round(cyc / secs / 1e9, 3), "cycles_per_instruction_of_first_wavefront": round(cyc / (float(self.instructions_per_iter) * self.iters), 2),
                "constant_rate_counter_khz": rate_khz}


class MfmaRateZeros(_MfmaIssueRate):
    name = "mfma_rate_zeros"
    operands = 0


class MfmaRateRandom(_MfmaIssueRate):
    name = "mfma_rate_random"
    operands = 2


class _Mfma16IssueRate(_MfmaIssueRate):
    """the same for v_mfma_f32_16x16x32_bf16, the instruction of the tiled GEMM on the fragment-ordered weight"""
    kernel = "probe_mfma_bf16_16x16_kernel"
    entry = "bench_probe_mfma_bf16_16x16"
    instruction = "v_mfma_f32_16x16x32_bf16"
    flop_per_instruction = 2.0 * 16 * 16 * 32
    nominal_cycles = 16
    instructions_per_iter = 16


class Mfma16RateZeros(_Mfma16IssueRate):
    name = "mfma16_rate_zeros"
    operands = 0


class Mfma16RateRandom(_Mfma16IssueRate):
    name = "mfma16_rate_random"
    operands = 2


class _MfmaF8F4Rate(_MfmaIssueRate):
    kernel = "probe_mfma_f8f4_kernel"
    entry = "bench_probe_mfma_f8f4"
    instruction = "v_mfma_scale_f32_32x32x64_f8f6f4 (e4m3 x e2m1, scales of 1)"
    flop_per_instruction = 2.0 * 32 * 32 * 64
    nominal_cycles = 64
    mfma_dtype = "fp8"
    dtype = "mxfp8 x mxfp4"
    iters = 2048
    random_kind = "random codes"


class MfmaF8F4RateZeros(_MfmaF8F4Rate):
    name = "mfma_f8f4_rate_zeros"
    operands = 0


class MfmaF8F4RateRandom(_MfmaF8F4Rate):
    name = "mfma_f8f4_rate_random"
    operands = 2


class MxintLinear(Workload):
    name = "mxint_linear"
    default_steps, default_warmup = 1000, 100
    metric = "MXINT8 Linear forward throughput (2*M*N*K flop per step; activation quantization included in the step)"
    unit = "TFLOP/s"
    dtype = "bf16"
    bound = "mfma"
    mfma_dtype = "bf16"
    kernel = "gemm_bf16_tn_kernel"
    M = N = K = 4096
    config = {"workload": "LinearMXInt 4096x4096 (bias zeros), x fp32 [4096,4096] N(0,1), W N(0,0.02), block 32, "
                          "8-bit mantissas; weights quantized at load_state_dict, seed 2"}
    cfg = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8}

    def make(self, torch):
        g = torch.Generator().manual_seed(2)
        x = torch.randn(self.M, self.K, generator=g)
        w = torch.randn(self.N, self.K, generator=g) * 0.02
        b = torch.zeros(self.N)
        return x, w, b

    def setup(self, torch, dev, n_buffers):
        from mase_amd.quantized import LinearMXInt
        from mase_amd.quantizers import _ops
        from mase_amd._gemm import gemm_bf16_tn

        self.torch = torch
        x, w, b = self.make(torch)
        self.host = (x, w, b)
        self.m = LinearMXInt(self.K, self.N, bias=True, device=dev, config=dict(self.cfg))
        self.m.load_state_dict({"weight": w, "bias": b})
        self.bufs = [x.to(dev).roll(i, dims=0).contiguous() for i in range(max(n_buffers, 4))]
        self.xq = _ops.mxint_qdq(self.bufs[0], 32, 8, -1, 8, out_dtype=torch.bfloat16)
        self.wb = self.m._w_cache.get(self.m.weight)
        assert self.wb is not None
        self.wp = self.m._w_cache.packed()  # the fragment-ordered copy the module's own forward uses
        self._gemm = gemm_bf16_tn

    def step(self, i):
        self.out = self.m(self.bufs[i % len(self.bufs)])

    def dominant_step(self, i):
        self.out = self._gemm(self.xq, self.wb, self.m.bias, self.torch.float32, b_packed=self.wp)

    def work_per_step(self):
        return 2.0 * self.M * self.N * self.K

    def cpu_baseline(self, torch, budget_s):
        from oracle import linear as OL

        x, w, b = self.host
        qw, qb = OL.mxint_prepare_weights(w, b, self.cfg)
        OL.linear_mxint_forward(x[:64], qw, qb, self.cfg)
        t0 = time.perf_counter()
        n = 0
        while True:
            OL.linear_mxint_forward(x, qw, qb, self.cfg)
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 20:
                break
        dt = (time.perf_counter() - t0) / n
        return {"value": self.work_per_step() / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                "kind": "port", "sample": f"{n} full forwards (activation quantize-dequantize + fp32 F.linear), {dt*1e3:.0f} ms each"}


class MxintLinearCodes(MxintLinear):
    """config 3's operands with the weight kept as fragment-ordered MXINT8 codes (1.03 B per weight) that the tiled
    kernel widens in registers: ``config["weight_memory"] = "codes"``"""
    name = "mxint_linear_codes"
    config = {"workload": MxintLinear.config["workload"] + "; weight_memory=codes"}

    def setup(self, torch, dev, n_buffers):
        from mase_amd.quantized import LinearMXInt
        from mase_amd.quantizers import _ops
        from mase_amd._gemm import gemm_mxint8_tn_packed

        self.torch = torch
        x, w, b = self.make(torch)
        self.host = (x, w, b)
        self.m = LinearMXInt(self.K, self.N, bias=True, device=dev, config=dict(self.cfg, weight_memory="codes"))
        self.m.load_state_dict({"weight": w, "bias": b})
        self.bufs = [x.to(dev).roll(i, dims=0).contiguous() for i in range(max(n_buffers, 4))]
        self.xq = _ops.mxint_qdq(self.bufs[0], 32, 8, -1, 8, out_dtype=torch.bfloat16)
        self.img = self.m._w_image
        assert self.img.valid_for(self.m.weight)
        self._gemm = gemm_mxint8_tn_packed

    def dominant_step(self, i):
        self.out = self._gemm(self.xq, self.img.codes, self.img.scales, self.img.n, self.m.bias, self.torch.float32)


class MxfpLinear(Workload):
    name = "mxfp_linear"
    default_steps, default_warmup = 300, 50
    metric = ("MXFP8 x MXFP4 Linear forward throughput (2*M*N*K flop per step; activation quantization to packed "
              "codes included in the step)")
    unit = "TFLOP/s"
    dtype = "fp8"
    bound = "mfma"
    mfma_dtype = "fp8"
    kernel = "gemm_mxfp_kernel"
    M, K, N = 8192, 8192, 28672
    config = {"workload": "LinearMXFP 8192->28672 (no bias), x bf16 [8192,8192] N(0,1) with 8 of 8192 channels x20, "
                          "W N(0,0.02); weights e2m1, activations e4m3, block 32, E8M0 scales; block-scaled MFMA, "
                          "fp32 accumulate, bf16 out; seed 3"}
    cfg = {"weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1,
           "data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}

    def make_x(self, torch, rows):
        g = torch.Generator().manual_seed(3)
        idx = torch.randperm(self.K, generator=g)[: self.K // 1000]
        x = torch.randn(rows, self.K, generator=g)
        x[:, idx] *= 20
        return x.to(torch.bfloat16)

    def make_w(self, torch, rows):
        g = torch.Generator().manual_seed(33)
        return (torch.randn(rows, self.K, generator=g) * 0.02).to(torch.bfloat16)

    def setup(self, torch, dev, n_buffers):
        from mase_amd.quantized import LinearMXFP
        from mase_amd._gemm import gemm_mxfp4_scaled_tiled, mxfp_pack_tiled

        self.torch = torch
        self.m = LinearMXFP(self.K, self.N, bias=False, device=dev, dtype=torch.bfloat16, config=dict(self.cfg))
        self.m.load_state_dict({"weight": self.make_w(torch, self.N)})
        assert self.m._w_packed.valid_for(self.m.weight)
        x = self.make_x(torch, self.M).to(dev)
        self.bufs = [x.roll(i, dims=0).contiguous() for i in range(max(n_buffers, 2))]
        self.xt, self.xs = mxfp_pack_tiled(self.bufs[0], 4, 3)
        self._gemm = gemm_mxfp4_scaled_tiled

    def step(self, i):
        self.out = self.m(self.bufs[i % len(self.bufs)])

    def dominant_step(self, i):
        p = self.m._w_packed
        self.out = self._gemm(self.xt, self.xs, (4, 3), p.tiled(self.K), p.scales, None, self.torch.bfloat16)

    def work_per_step(self):
        return 2.0 * self.M * self.N * self.K

    def cpu_baseline(self, torch, budget_s):
        from oracle import linear as OL

        ms, ns = 1024, 4096  # bounded sample: the first 1024 activation rows against the first 4096 weight rows
        x = self.make_x(torch, ms)
        qw, _ = OL.mxfp_prepare_weights(self.make_w(torch, ns), None, self.cfg)
        OL.linear_mxfp_forward(x[:64], qw, None, self.cfg)
        t0 = time.perf_counter()
        n = 0
        while True:
            OL.linear_mxfp_forward(x, qw, None, self.cfg)
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 20:
                break
        dt = (time.perf_counter() - t0) / n
        return {"value": 2.0 * ms * ns * self.K / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                "kind": "port", "sample": f"{n} forwards of a [{ms},{self.K}] x [{ns},{self.K}] slice of the workload "
                                          f"(activation quantize-dequantize + bf16 F.linear), {dt*1e3:.0f} ms each"}


class DecoderLayerMxint(Workload):
    name = "decoder_layer"
    default_steps, default_warmup = 100, 10
    metric = ("Llama-style decoder layer forward with MXINT8 Linears (flop per step = 7 Linears + causal attention; "
              "RMSNorm, rotary embedding, the SwiGLU product and causal attention run as one-pass kernels of this "
              "library, all inside the step)")
    unit = "TFLOP/s"
    dtype = "bf16"
    bound = "mfma"
    mfma_dtype = "bf16"
    kernel = "gemm_bf16_tn_kernel"
    B, T = 8, 2048
    config = {"workload": "decoder layer hidden 4096, 32 heads x 128, SwiGLU 11008, RMSNorm eps 1e-6, RoPE theta 1e4, "
                          "causal, batch 8 x seq 2048, bf16, weights N(0,0.02) seed 40, x N(0,1) seed 4; every nn.Linear "
                          "-> LinearMXInt (block 32, 8-bit) through quantize_module_transform_pass"}
    cfg = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8}

    def build(self, torch, device):
        from mase_amd.workloads import DecoderLayer, DecoderLayerConfig

        return DecoderLayer(DecoderLayerConfig(), device=device, dtype=torch.bfloat16, seed=40)

    def setup(self, torch, dev, n_buffers):
        from mase_amd.passes import quantize_module_transform_pass
        from mase_amd.quantizers import _ops
        from mase_amd._gemm import gemm_bf16_tn

        self.torch = torch
        layer = self.build(torch, dev)
        self.layer, _ = quantize_module_transform_pass(
            layer, {"by": "type", "linear": {"config": dict(self.cfg, name="mxint")}})
        x = torch.randn(self.B, self.T, 4096, generator=torch.Generator().manual_seed(4)).bfloat16().to(dev)
        self.bufs = [x.roll(i, dims=1).contiguous() for i in range(max(n_buffers, 2))]
        # operands of the seven contractions alone, for the kernel-only timing
        tok = self.B * self.T
        a4096 = _ops.mxint_qdq(self.bufs[0].reshape(tok, 4096), 32, 8, -1, 8, out_dtype=torch.bfloat16)
        a11008 = _ops.mxint_qdq(torch.randn(tok, 11008, device=dev, dtype=torch.bfloat16), 32, 8, -1, 8,
                                out_dtype=torch.bfloat16)
        self.gemms = []
        for name in ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"):
            m = getattr(self.layer, name)
            wb = m._w_cache.get(m.weight)
            assert wb is not None
            self.gemms.append((a11008 if name == "down_proj" else a4096, wb, m._w_cache.packed()))
        self._gemm = gemm_bf16_tn
        self.linear_flops = self.layer.linear_flops(tok)
        self.attn_flops = 4.0 * self.B * 32 * self.T * self.T * 128 / 2  # causal: half of the score matrix

    def step(self, i):
        with self.torch.no_grad():
            self.out = self.layer(self.bufs[i % len(self.bufs)])

    def dominant_step(self, i):
        for a, w, wp in self.gemms:  # as the modules' own forwards call it
            self.out = self._gemm(a, w, None, self.torch.bfloat16, b_packed=wp)

    def work_per_step(self):
        return self.linear_flops + self.attn_flops

    def dominant_work(self):
        return self.linear_flops

    def cpu_baseline(self, torch, budget_s):
        from oracle import linear as OL

        class _OracleLinear(torch.nn.Module):
            def __init__(self, qw, cfg):
                super().__init__()
                self.qw, self.cfg = qw, cfg

            def forward(self, x):
                return OL.linear_mxint_forward(x, self.qw, None, self.cfg)

        layer = self.build(torch, None)
        for name, m in list(layer.named_children()):
            if isinstance(m, torch.nn.Linear):
                qw, _ = OL.mxint_prepare_weights(m.weight.data, None, self.cfg)
                setattr(layer, name, _OracleLinear(qw, self.cfg))
        tokens = 128
        x = torch.randn(1, tokens, 4096, generator=torch.Generator().manual_seed(4)).bfloat16()
        with torch.no_grad():
            layer(x[:, :16])
            t0 = time.perf_counter()
            n = 0
            while True:
                layer(x)
                n += 1
                if time.perf_counter() - t0 > budget_s or n >= 20:
                    break
        dt = (time.perf_counter() - t0) / n
        flops = layer.linear_flops(tokens) + 4.0 * 32 * tokens * tokens * 128 / 2
        return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"{n} forwards of the same layer on 1 x {tokens} tokens (bf16, reference Linear forward), "
                          f"{dt*1e3:.0f} ms each"}


class _ElementwiseQdq(Workload):
    """the element-wise / per-block quantizers on a tensor of config 2's size ([8,2048,4096], N(0,1), seed 5) in the
    dtype given by --dtype (default bf16)"""
    shape = (8, 2048, 4096)
    torch_dtype = None
    fn_name = ""
    args = ()

    def setup(self, torch, dev, n_buffers):
        import mase_amd.quantizers as Q

        self.fn = getattr(Q, self.fn_name)
        g = torch.Generator().manual_seed(5)
        self.host = torch.randn(*self.shape, generator=g).to(self.torch_dtype)
        self.bufs = [self.host.to(dev).roll(i, dims=1).contiguous() for i in range(n_buffers)]
        self.dtype = {torch.bfloat16: "bf16", torch.float32: "f32", torch.float16: "f16"}[self.torch_dtype]
        if self.torch_dtype != torch.float32 and getattr(self, "kernel16", None):
            self.kernel = self.kernel16
        self.config = {"workload": f"{self.fn_name}{self.args} on {self.dtype} {list(self.shape)}, N(0,1) seed 5"}
        self.metric = (f"{self.fn_name} throughput (algorithmic bytes: {self.host.element_size()} B read + "
                       f"{self.host.element_size()} B written per element)")

    def step(self, i):
        self.out = self.fn(self.bufs[i % len(self.bufs)], *self.args)

    def work_per_step(self):
        return float(self.host.numel() * 2 * self.host.element_size())

    def cpu_baseline(self, torch, budget_s):
        import oracle as O

        fn = getattr(O, self.oracle_name)
        x = self.host[:1].contiguous()  # one of the 8 batch items
        fn(x[:, :64].contiguous(), *self.oracle_args)
        t0 = time.perf_counter()
        n = 0
        while True:
            fn(x, *self.oracle_args)
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 20:
                break
        dt = (time.perf_counter() - t0) / n
        return {"value": self.work_per_step() / 8 / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                "kind": "port", "sample": f"{n} passes over one batch item [1,2048,4096], {dt*1e3:.0f} ms each"}


class IntegerQdq(_ElementwiseQdq):
    name, unit, kernel = "integer_qdq", "GB/s", "elementwise_kernel<IntegerOp>"
    fn_name, args = "integer_quantizer", (8, 4)
    oracle_name, oracle_args = "integer_quantizer", (8, 4)


class MinifloatDenormQdq(_ElementwiseQdq):
    name, unit, kernel = "minifloat_denorm_qdq", "GB/s", "minifloat_value_kernel"
    fn_name, args = "minifloat_denorm_quantizer", (8, 4, None)
    oracle_name, oracle_args = "minifloat_denorm_quantizer", (8, 4, None)


class MinifloatIeeeQdq(_ElementwiseQdq):
    name, unit, kernel = "minifloat_ieee_qdq", "GB/s", "minifloat_value_kernel"
    fn_name, args = "minifloat_ieee_quantizer", (8, 4, None)
    oracle_name, oracle_args = "minifloat_ieee_quantizer", (8, 4, None)


class MxfpQdq(_ElementwiseQdq):
    name, unit, kernel = "mxfp_qdq", "GB/s", "mxfp_qdq_vec_kernel"
    kernel16 = "mxfp_qdq_pk16_kernel"
    fn_name, args = "mxfp_quantizer", (32, 4, 3)
    oracle_name, oracle_args = "mxfp_quantizer", (32, 4, 3)


class MxintClipSearch(_ElementwiseQdq):
    """mxint_quantizer(quantile_search=True): 11 candidate scales per block of 32, the weight-loading path of LinearMXInt
    with config["clip_search"]"""
    default_steps, default_warmup = 1000, 100
    name, unit, kernel = "mxint_clip_search", "GB/s", "mxint_clip_search_kernel"
    fn_name, args = "mxint_quantizer", (32, 4, -1, 8, True)
    oracle_name, oracle_args = "mxint_quantizer", (32, 4, -1, 8, True)


class MinifloatMxQdq(_ElementwiseQdq):
    name, unit, kernel = "minifloat_mx_qdq", "GB/s", "elementwise_kernel<MinifloatMxOp>"
    kernel16 = "minifloat_mx_pk16_kernel"
    oracle_name, oracle_args = "minifloat_quantizer_sim", (4, 3, True, "rn")

    def setup(self, torch, dev, n_buffers):
        import mase_amd.quantizers as Q

        self.fn_name = "minifloat_quantizer_sim"
        super().setup(torch, dev, n_buffers)
        meta = Q.MinifloatMeta(exp_bits=4, frac_bits=3, is_finite=True, round_mode="rn")
        self.fn = lambda t: Q.minifloat_quantizer_sim(t, meta)
        self.config = {"workload": f"minifloat_quantizer_sim e4m3 finite rn on {self.dtype} {list(self.shape)}, N(0,1) seed 5"}


class AttnProb(Workload):
    """score -> probability chain of the MX-quantized Llama attention (scale, causal mask, minifloat cast e5m8,
    fp32 softmax, MXINT8 blocks of 32) on [4,32,2048,2048]"""
    default_steps, default_warmup = 300, 50
    name = "attn_prob"
    unit = "GB/s"
    kernel = "attn_prob_kernel"
    shape = (4, 32, 2048, 2048)
    torch_dtype = None

    def setup(self, torch, dev, n_buffers):
        from mase_amd.quantizers._ops import attn_softmax_mx

        self.op = attn_softmax_mx
        B, H, S, T = self.shape
        dt = self.torch_dtype
        self.dtype = {torch.bfloat16: "bf16", torch.float32: "f32", torch.float16: "f16"}[dt]
        g = torch.Generator(device=dev).manual_seed(6)
        self.bufs = [(torch.randn(B, H, S, T, device=dev, generator=g) * 4).to(dt) for _ in range(max(2, min(n_buffers, 3)))]
        self.mask = torch.triu(torch.full((S, T), torch.finfo(dt).min, dtype=dt, device=dev), diagonal=1)[None, None] \
            .expand(B, 1, S, T).contiguous()
        self.esize = self.bufs[0].element_size()
        self.metric = (f"attention probability chain throughput (algorithmic bytes: {self.esize} B of scores read + "
                       f"{self.esize} B of probabilities written per element)")
        self.config = {"workload": f"scores {self.dtype} {list(self.shape)} N(0,16) seed 6, scaling 0.0884, causal mask, "
                                   "cast e5m8, softmax, MXINT8 block 32"}

    def step(self, i):
        self.out = self.op(self.bufs[i % len(self.bufs)], self.mask, 0.0884, (5, 8, True, "rn"), ("mxint", 8))

    def work_per_step(self):
        B, H, S, T = self.shape
        return float(B * H * S * T * 2 * self.esize)

    def cpu_baseline(self, torch, budget_s):
        import oracle as O

        x = self.bufs[0][0, :2].cpu()[None]           # 2 heads of one batch item
        m = self.mask[:1].cpu()
        t0 = time.perf_counter()
        n = 0
        while True:
            w = x * 0.0884 + m
            w = O.minifloat_quantizer_sim(w, 5, 8, True, "rn")
            w = torch.softmax(w.to(torch.float32), dim=-1).to(x.dtype)
            O.mxint_quantizer(w, 32, 8, block_dim=-1)
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 10:
                break
        dt = (time.perf_counter() - t0) / n
        return {"value": x.numel() * 2 * self.esize / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                "kind": "port", "sample": f"{n} passes of the separate tensor operations over 2 heads [1,2,2048,2048], {dt*1e3:.0f} ms each"}


class BmmScores(Workload):
    """the score product of a quantized attention block on its own: q [8, 32, 2048, 128] (a view of [batch, tokens,
    heads, 128] memory, already MXINT8-quantized along the head dimension) times k^T, bf16 scores written to memory:
    mase_gemm_bf16_tn_batched.  Bound by writing the [2048, 2048] score matrix of every head."""
    name = "bmm_scores"
    default_steps, default_warmup = 100, 10
    unit = "GB/s"
    dtype = "bf16"
    kernel = "gemm_bf16_tn_kernel"
    shape = (8, 32, 2048, 128)
    metric = ("batched score product q k^T of an attention block (algorithmic bytes: 2 B per operand element read + 2 B "
              "per score written)")
    config = {"workload": "q, k bf16 [8,32,2048,128] as views of [batch, tokens, heads, 128], MXINT8 values, seed 9; scores "
                          "bf16 [8,32,2048,2048]"}

    def setup(self, torch, dev, n_buffers):
        from mase_amd._gemm import gemm_bf16_tn_batched
        from mase_amd.quantizers import _ops

        self.op = gemm_bf16_tn_batched
        B, H, T, D = self.shape
        g = torch.Generator(device=dev).manual_seed(9)
        mk = lambda: _ops.mxint_qdq(torch.randn(B, T, H, D, device=dev, generator=g).bfloat16(), 32, 8, -1, 8).transpose(1, 2)
        self.sets = [(mk(), mk()) for _ in range(2)]
        self.outs = [torch.empty(B, H, T, T, dtype=torch.bfloat16, device=dev) for _ in range(2)]

    def step(self, i):
        q, k = self.sets[i % 2]
        self.out = self.op(q, k, out=self.outs[i % 2])

    def work_per_step(self):
        B, H, T, D = self.shape
        return float(2 * B * H * T * D * 2 + B * H * T * T * 2)

    def cpu_baseline(self, torch, budget_s):
        q, k = (t[:1, :2].float().cpu() for t in self.sets[0])  # 2 heads of one batch item
        t0 = time.perf_counter()
        n = 0
        while True:
            torch.matmul(q, k.transpose(-1, -2))
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 50:
                break
        dt = (time.perf_counter() - t0) / n
        T, D = self.shape[2], self.shape[3]
        return {"value": 2 * (2 * T * D * 4 + T * T * 4) / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"{n} torch.matmul calls over 2 heads in fp32 (bytes counted at 4 B per element), {dt*1e3:.1f} ms each"}


class AttentionCausal(Workload):
    """the decoder layer's attention core on its own: causal softmax(q k^T / sqrt(d)) v, bf16, batch 8 x 32 heads x 2048
    tokens x 128, operands as strided views of [batch, tokens, heads, 128] memory (what the projections produce)"""
    name = "attention_causal"
    default_steps, default_warmup = 200, 20
    unit = "TFLOP/s"
    dtype = "bf16"
    bound = "mfma"
    kernel = "attn_causal_fwd_kernel"
    shape = (8, 32, 2048, 128)

    def setup(self, torch, dev, n_buffers):
        from mase_amd.quantizers import _ops

        self._ops = _ops
        B, H, T, D = self.shape
        g = torch.Generator(device=dev).manual_seed(7)
        mk = lambda: torch.randn(B, T, H, D, device=dev, generator=g).bfloat16().transpose(1, 2)
        self.sets = [(mk(), mk(), mk()) for _ in range(2)]
        self.metric = "causal attention core throughput (4 * batch * heads * tokens^2 * 128 / 2 flop per step: the unmasked half)"
        self.config = {"workload": f"q, k, v bf16 {list(self.shape)} N(0,1) seed 7, scaling 128^-0.5, causal"}

    def step(self, i):
        q, k, v = self.sets[i % 2]
        self.out = self._ops.attention_causal(q, k, v)

    def work_per_step(self):
        B, H, T, D = self.shape
        return 4.0 * B * H * T * T * D / 2

    def cpu_baseline(self, torch, budget_s):
        B, H, T, D = self.shape
        q, k, v = (t[:1, :2].float().cpu() for t in self.sets[0])  # 2 heads of one batch item
        mask = torch.triu(torch.ones(T, T, dtype=torch.bool), 1)
        t0 = time.perf_counter()
        n = 0
        while True:
            s = (q @ k.transpose(-1, -2)) * D ** -0.5
            torch.softmax(s.masked_fill(mask, float("-inf")), -1) @ v
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 20:
                break
        dt = (time.perf_counter() - t0) / n
        return {"value": 4.0 * 2 * T * T * D / 2 / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"{n} passes of the tensor operations (fp32, full score matrix) over 2 heads, {dt*1e3:.0f} ms each; "
                          "flop counted as for the GPU (the unmasked half)"}


class DecodeLinear(Workload):
    """LinearMXInt forward for a handful of tokens: bound by streaming the weight once"""
    name = "decode_linear"
    unit = "GB/s"
    dtype = "bf16"
    kernel = "gemm_skinny_partial_kernel"
    M, N, K = 16, 28672, 8192
    metric = "MXINT8 Linear forward for 16 tokens (algorithmic bytes: the bf16 weight image, 2 B per weight, read once)"
    config = {"workload": "LinearMXInt 8192 -> 28672, 16 tokens, bf16, weights N(0,0.02) seed 7"}
    extra_cfg = {}
    weight_bytes = 2.0

    def setup(self, torch, dev, n_buffers):
        from mase_amd.quantized import LinearMXInt

        cfg = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8, **self.extra_cfg}
        g = torch.Generator().manual_seed(7)
        self.mods = []
        for i in range(2):  # two layers, alternated: the 470 MB weight cannot stay in the last-level cache
            m = LinearMXInt(self.K, self.N, bias=False, device=dev, dtype=torch.bfloat16, config=dict(cfg))
            m.load_state_dict({"weight": (torch.randn(self.N, self.K, generator=g) * 0.02).bfloat16()})
            self.mods.append(m)
        self.x = torch.randn(self.M, self.K, generator=g).bfloat16().to(dev)

    def step(self, i):
        self.out = self.mods[i % 2](self.x)

    def work_per_step(self):
        return float(self.N * self.K) * self.weight_bytes

    def cpu_baseline(self, torch, budget_s):
        from oracle import linear as OL

        cfg = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8}
        n_rows = 2048
        w = self.mods[0].weight.data[:n_rows].float().cpu()
        x = self.x.float().cpu()
        t0 = time.perf_counter()
        n = 0
        while True:
            OL.linear_mxint_forward(x, w, None, cfg)
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 20:
                break
        dt = (time.perf_counter() - t0) / n
        return {"value": n_rows * self.K * self.weight_bytes / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"{n} forwards with {n_rows} of the {self.N} output rows (fp32 on the CPU), {dt*1e3:.0f} ms each"}


class DecodeLinearPacked(DecodeLinear):
    """the same forward with the weight streamed as MXINT8 codes + scale bytes (config packed_decode)"""
    name = "decode_linear_packed"
    kernel = "gemm_skinny_mxint8_shared_kernel"
    metric = ("MXINT8 Linear forward for 16 tokens, weight streamed as int8 codes + scale bytes (algorithmic bytes: "
              "1.03125 B per weight, read once)")
    config = {"workload": "LinearMXInt 8192 -> 28672 with packed_decode, 16 tokens, bf16, weights N(0,0.02) seed 7"}
    extra_cfg = {"packed_decode": True}
    weight_bytes = 1.03125


class DecodeLinearMxfp4(Workload):
    """LinearMXFP (e2m1 weights, e4m3 activations) forward for a handful of tokens: the weight codes streamed once"""
    name = "decode_linear_mxfp4"
    unit = "GB/s"
    dtype = "fp8"
    kernel = "gemm_skinny_mxfp4_shared_kernel"
    M, N, K = 16, 28672, 8192
    metric = ("MXFP4-weight Linear forward for 16 tokens (algorithmic bytes: e2m1 codes + E8M0 scales, 0.53125 B per "
              "weight, read once)")
    config = {"workload": "LinearMXFP 8192 -> 28672 (e2m1 weights, e4m3 activations, block 32), 16 tokens, bf16, "
                          "weights N(0,0.02) seed 7"}
    cfg = {"weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1,
           "data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}

    def setup(self, torch, dev, n_buffers):
        from mase_amd.quantized import LinearMXFP

        g = torch.Generator().manual_seed(7)
        self.mods = []
        for i in range(3):  # alternated layers: 3 x 125 MB of codes, beyond what the last-level cache keeps hot
            m = LinearMXFP(self.K, self.N, bias=False, device=dev, dtype=torch.bfloat16, config=dict(self.cfg))
            m.load_state_dict({"weight": (torch.randn(self.N, self.K, generator=g) * 0.02).bfloat16()})
            assert m._w_packed.valid_for(m.weight)
            self.mods.append(m)
        self.x = torch.randn(self.M, self.K, generator=g).bfloat16().to(dev)

    def step(self, i):
        self.out = self.mods[i % 3](self.x)

    def work_per_step(self):
        return float(self.N * self.K) * 0.53125

    def cpu_baseline(self, torch, budget_s):
        from oracle import linear as OL

        n_rows = 2048
        w = self.mods[0].weight.data[:n_rows].float().cpu()
        x = self.x.float().cpu()
        t0 = time.perf_counter()
        n = 0
        while True:
            OL.linear_mxfp_forward(x, w, None, self.cfg)
            n += 1
            if time.perf_counter() - t0 > budget_s or n >= 20:
                break
        dt = (time.perf_counter() - t0) / n
        return {"value": n_rows * self.K * 0.53125 / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                "kind": "port", "sample": f"{n} forwards with {n_rows} of the {self.N} output rows (fp32 on the CPU), {dt*1e3:.0f} ms each"}


WORKLOADS = {w.name: w for w in (MxintClipSearch, BfpQdq, MxintQdq, MxintLinear, MxintLinearCodes, MxfpLinear, DecoderLayerMxint, CopyBytes, IntegerQdq,
                                 MinifloatDenormQdq, MinifloatIeeeQdq, MinifloatMxQdq, MxfpQdq, AttnProb, DecodeLinear,
                                 DecodeLinearPacked, DecodeLinearMxfp4, AttentionCausal, BmmScores, MfmaRateZeros, MfmaRateRandom, Mfma16RateZeros, Mfma16RateRandom, MfmaF8F4RateZeros,
                                 MfmaF8F4RateRandom)}


def load_traffic(name):
    """HBM bytes per launch of the dominant kernel, measured beforehand with rocprofv3 --pmc (FETCH_SIZE / WRITE_SIZE,
    two separate runs) and committed as a summary; None when there is none.  It is not measured by this run."""
    rel = os.path.join("profiles", f"traffic_{name}.json")
    path = os.path.join(ROOT, rel)
    if os.path.exists(path):
        with open(path) as f:
            return json.load(f).get("traffic_bytes_per_launch"), rel
    return None, None


HEADLINE = ("bfp_qdq", "mxint_qdq", "mxint_linear", "mxfp_linear", "decoder_layer")  # configs 2, 1, 3, 4, 5
REGIONS = 5             # timed regions per workload; the median is reported
SETTLE_SECONDS = 0.06  # untimed run-in before the warm-up steps, so that clocks and memory system are at steady state


def measure(torch, dev, name, steps, warmup, a):
    """One workload: W warm-up steps, REGIONS regions of K wall-clock-timed steps each bracketed by synchronisation
    (median reported), as many event-timed regions of K launches of the dominant kernel, the CPU baseline leg.
    Returns the fields of a bench line for it."""
    w = WORKLOADS[name]()
    steps = w.default_steps if steps is None else steps
    warmup = w.default_warmup if warmup is None else warmup
    if hasattr(w, "torch_dtype"):
        w.torch_dtype = {"bf16": torch.bfloat16, "f32": torch.float32, "f16": torch.float16}[a.dtype]
    w.setup(torch, dev, a.buffers)
    # run-in (not counted as steps): short timed regions otherwise read the ramp of the clocks, not the kernel
    t0 = time.perf_counter()
    settle = 0
    while time.perf_counter() - t0 < SETTLE_SECONDS:
        w.step(settle)
        settle += 1
        if settle % 16 == 0:
            torch.cuda.synchronize()
    for i in range(warmup):
        w.step(i)
    torch.cuda.synchronize()

    # whole-job timing: REGIONS regions of exactly `steps` steps each, every region bracketed by synchronisation and
    # timed on the wall clock; the median region is reported (a region of 20 steps of a 40 us kernel lasts under a
    # millisecond, and a single such reading moves by several per cent)
    walls = []
    for _ in range(REGIONS):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            w.step(i)
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t0)
    wall = sorted(walls)[REGIONS // 2]

    # kernel timing: a HIP event pair on the launch stream (torch's current stream is the one handed to the C ABI)
    # around `steps` back-to-back launches of the dominant kernel; average launch duration = elapsed / steps; the
    # median of REGIONS such regions
    dominant = getattr(w, "dominant_step", w.step)
    k_regions = []
    for _ in range(REGIONS):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            dominant(i)
        e1.record()
        torch.cuda.synchronize()
        k_regions.append(e0.elapsed_time(e1) / steps)
    k_avg = sorted(k_regions)[REGIONS // 2]

    work = w.work_per_step()
    scale = 1e9 if w.bound == "hbm" else 1e12
    value = work * steps / wall / scale
    dominant_work = w.dominant_work() if hasattr(w, "dominant_work") else work
    achieved = dominant_work / (k_avg * 1e-3) / scale
    peak = HBM_PEAK_GBS if w.bound == "hbm" else MFMA_PEAK_TFLOPS[getattr(w, "mfma_dtype", "bf16")]
    traffic, traffic_src = load_traffic(w.name)
    cpu = None if a.no_cpu else w.cpu_baseline(torch, a.cpu_seconds)
    out = {
        "workload": w.name,
        "metric": w.metric,
        "value": round(value, 2),
        "unit": w.unit,
        "steps": steps,
        "warmup": warmup,
        "settle_steps": settle,
        "ms_per_step": round(wall / steps * 1e3, 5),
        "timed_regions": REGIONS,
        "ms_per_step_regions": [round(t / steps * 1e3, 5) for t in walls],
        "whole_step_frac": round(value / peak, 4),
        "dtype": w.dtype,
        "config": w.config,
        "roofline": {
            "bound": w.bound,
            "kernel": w.kernel,
            "achieved": round(achieved, 2),
            "peak": peak,
            "unit": "GB/s" if w.bound == "hbm" else "TFLOP/s",
            "frac": round(achieved / peak, 4),
            "traffic": traffic,
            "traffic_source": traffic_src,
            "kernel_ms_avg": round(k_avg, 5),
        },
        "cpu_baseline": cpu,
    }
    # where the dominant kernel is the whole step, its average launch cannot take longer than a step
    if not hasattr(w, "dominant_step"):
        ok = k_avg <= wall / steps * 1e3 * 1.01
        out["consistency"] = {"kernel_ms_avg_le_ms_per_step": bool(ok)}
        if not ok:
            out["warning"] = (f"dominant kernel average {k_avg:.5f} ms exceeds the whole step {wall / steps * 1e3:.5f} ms: the "
                              "timed regions are too short to resolve; rerun with more --steps")
    if hasattr(w, "extra"):
        out["extra"] = w.extra(torch)
    del w
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default: the workload's own)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed warm-up steps (default: the workload's own)")
    ap.add_argument("--workload", default="all", choices=["all"] + sorted(WORKLOADS),
                    help="all (default): the five headline configurations, config 2 as the headline of the line")
    ap.add_argument("--buffers", type=int, default=4)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f32", "f16"],
                    help="tensor dtype of the secondary workloads (the headline ones fix theirs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=None,
                    help="budget of each CPU baseline leg (default 15 for one workload, 6 each for all)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); multi-GPU sharding is a design note, not code",
              file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no ROCm device visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if a.cpu_seconds is None:
        a.cpu_seconds = 6.0 if a.workload == "all" else 15.0
    names = HEADLINE if a.workload == "all" else (a.workload,)
    results = []
    for i, name in enumerate(names):
        # --steps / --warmup apply to the headline workload; the other configurations of `all` run their own counts
        # (stated in their entries), sized so that each timed region lasts tens of milliseconds
        r = measure(torch, dev, name, a.steps if i == 0 else None, a.warmup if i == 0 else None, a)
        print(f"bench.py: {name}: {r['value']} {r['unit']} whole step ({r['whole_step_frac']:.3f} of peak), dominant "
              f"kernel {r['roofline']['frac']:.3f} of peak", file=sys.stderr, flush=True)
        results.append(r)
    head = results[0]
    out = {
        "metric": head["metric"],
        "value": head["value"],
        "unit": head["unit"],
        "n_gpus": 1,
        "steps": head["steps"],
        "warmup": head["warmup"],
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic",
        "config": head["config"],
        "roofline": head["roofline"],
        "cpu_baseline": head["cpu_baseline"],
        "settle_steps": head["settle_steps"],
        "timed_regions": head["timed_regions"],
        "ms_per_step_regions": head["ms_per_step_regions"],
        "whole_step_frac": head["whole_step_frac"],
    }
    for key in ("consistency", "warning"):
        if key in head:
            out[key] = head[key]
    if "extra" in head:
        out["extra"] = head["extra"]
    if a.workload == "all":
        out["configs"] = results
    print(json.dumps(out))


if __name__ == "__main__":
    main()
