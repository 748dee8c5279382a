"""CPU-side checks of the C-ABI library and of the host logic (no GPU, no kernel launches)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from mase_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__ as g

        g.build()
    return _lib.load()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mase_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mase_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    from mase_amd import _lib

    names = declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/mase_amd.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature in mase_amd/_lib.py"
    assert sorted(_lib.SIGNATURES) == names
    assert lib.mase_abi_version() >= 1
    assert lib.mase_error_string(0) == b"ok" and b"NULL" in lib.mase_error_string(-1)


def test_entry_points_reject_bad_arguments_without_a_gpu(lib):
    """argument validation happens before any HIP call, so it can be exercised on the CPU"""
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.mase_mxint_qdq(None, p, None, None, 64, 0, 0, 32, 8, 8, p, None) == -1
    assert lib.mase_mxint_qdq(p, p, None, None, 65, 0, 0, 32, 8, 8, p, None) == -2
    assert lib.mase_mxint_qdq(p, p, None, None, 64, 7, 0, 32, 8, 8, p, None) == -4
    assert lib.mase_mxint_qdq(p, p, None, None, 64, 0, 9, 32, 8, 8, p, None) == -4
    assert lib.mase_mxint_qdq(p, p, None, None, 64, 0, 0, 32, 1, 8, p, None) == -5
    assert lib.mase_mxint_qdq(p, p, p, None, 64, 0, 0, 32, 8, 8, p, None) == -1
    assert lib.mase_mxint_qdq(p, p, None, None, 0, 0, 0, 32, 8, 8, p, None) == 0  # empty input is a no-op
    assert lib.mase_gemm_bf16_tn(p, p, None, p, 4, 4, 96, 0, 0, None) == -2  # K must be whole 64-wide tiles
    assert lib.mase_gemm_bf16_tn(p, None, None, p, 4, 4, 64, 0, 0, None) == -1
    # mase_gemm_bf16_skinny(A, B, bias, C, M, N, K, out_dtype, bias_dtype, workspace, workspace_bytes, stream)
    assert lib.mase_gemm_bf16_skinny(p, p, None, p, 4, 4, 96, 0, 0, p, 4096, None) == -2     # K in whole 64-chunks
    assert lib.mase_gemm_bf16_skinny(p, p, None, p, 129, 4, 64, 0, 0, p, 4096, None) == -2   # at most 128 rows
    assert lib.mase_gemm_bf16_skinny(None, p, None, p, 4, 4, 64, 0, 0, p, 4096, None) == -1
    assert lib.mase_gemm_bf16_skinny(p, p, None, p, 4, 4, 64, 5, 0, p, 4096, None) == -4
    assert lib.mase_gemm_bf16_skinny_workspace_bytes(129, 4096, 4096) == 0   # outside the kernel's domain
    assert lib.mase_gemm_bf16_skinny_workspace_bytes(32, 4096, 100) == 0
    # mase_gemm_bf16_tn_splitk falls back to the plain entry point's checks when nothing is split (no device here)
    assert lib.mase_gemm_bf16_tn_splitk(p, p, None, p, 4, 4, 96, 0, 0, None, 0, None) == -2
    assert lib.mase_gemm_bf16_tn_splitk(p, None, None, p, 4, 4, 64, 0, 0, None, 0, None) == -1
    assert lib.mase_gemm_bf16_tn_splitk_workspace_bytes(0, 4, 64) == 0
    # mase_gemm_bf16_tn_packed(A, B_packed, bias, C, M, N, K, out_dtype, bias_dtype, stream) and the packer
    assert lib.mase_gemm_bf16_tn_packed(p, p, None, p, 256, 256, 192, 0, 0, None) == -2   # K in pairs of 64-element tiles
    assert lib.mase_gemm_bf16_tn_packed(p, None, None, p, 256, 256, 128, 0, 0, None) == -1
    assert lib.mase_gemm_bf16_tn_packed(p, p, None, p, 256, 256, 128, 4, 0, None) == -4
    assert lib.mase_gemm_bf16_tn_packed(p, p, None, p, 0, 256, 128, 0, 0, None) == 0
    assert lib.mase_gemm_bf16_pack_b(p, p, 64, 24, None) == -2
    assert lib.mase_gemm_bf16_pack_b(None, p, 64, 32, None) == -1
    assert lib.mase_gemm_bf16_packed_bytes(33, 64) == 64 * 64 * 2 and lib.mase_gemm_bf16_packed_bytes(32, 24) == 0
    # mase_gemm_mxfp4_scaled_tiled(A_tiled, A_scales, a_format, B_tiled, B_scales, bias, C, M, N, K, out_dtype,
    # bias_dtype, stream), the image maker and the activation quantizer that writes the image
    assert lib.mase_gemm_mxfp4_scaled_tiled(p, p, 0, p, p, None, p, 256, 256, 192, 0, 0, None) == -2  # K % 128
    assert lib.mase_gemm_mxfp4_scaled_tiled(p, p, 0, None, p, None, p, 256, 256, 512, 0, 0, None) == -1
    assert lib.mase_gemm_mxfp4_scaled_tiled(p, p, 0, p, p, None, p, 256, 256, 512, 3, 0, None) == -4
    assert lib.mase_gemm_mxfp4_scaled_tiled(p, p, 4, p, p, None, p, 256, 256, 512, 0, 0, None) == -5  # A must be 8-bit
    assert lib.mase_gemm_mxfp4_scaled_tiled(p, p, 0, p, p, None, p, 1 << 20, 256, 1 << 13, 0, 0, None) == -2  # image >= 2^32
    assert lib.mase_gemm_mxfp4_scaled_tiled(p, p, 0, p, p, None, p, 0, 256, 512, 0, 0, None) == 0
    assert lib.mase_mxfp_tile_codes(p, p, 64, 96, 4, None) == -2
    assert lib.mase_mxfp_tile_codes(p, p, 64, 128, 6, None) == -5
    assert lib.mase_mxfp_tile_codes(None, p, 64, 128, 4, None) == -1
    assert lib.mase_mxfp_tiled_bytes(257, 128, 4) == 512 * 64 and lib.mase_mxfp_tiled_bytes(257, 128, 8) == 512 * 128
    assert lib.mase_mxfp_tiled_bytes(256, 96, 8) == 0 and lib.mase_mxfp_tiled_bytes(256, 128, 6) == 0
    assert lib.mase_mxfp_pack_tiled(p, p, p, 4, 96, 0, 4, 3, p, None) == -2
    assert lib.mase_mxfp_pack_tiled(p, p, p, 4, 128, 0, 2, 1, p, None) == -5   # 8-bit element formats only
    assert lib.mase_mxfp_pack_tiled(p, p, p, 4, 128, 7, 4, 3, p, None) == -4
    assert lib.mase_mxfp_pack_tiled(p, None, p, 4, 128, 0, 4, 3, p, None) == -1
    # mase_gemm_mxint8_skinny(A, codes, scales, bias, C, M, N, K, out_dtype, bias_dtype, workspace, workspace_bytes, stream)
    assert lib.mase_gemm_mxint8_skinny(p, p, p, None, p, 4, 4, 192, 0, 0, p, 4096, None) == -2    # K in whole 128-chunks
    assert lib.mase_gemm_mxint8_skinny(p, p, p, None, p, 129, 4, 128, 0, 0, p, 4096, None) == -2
    assert lib.mase_gemm_mxint8_skinny(p, p, None, None, p, 4, 4, 128, 0, 0, p, 4096, None) == -1
    assert lib.mase_gemm_mxint8_skinny(p, p, p, None, p, 4, 4, 128, 9, 0, p, 4096, None) == -4
    assert lib.mase_gemm_mxint8_skinny_workspace_bytes(4, 4, 192) == 0
    # mase_gemm_mxfp4_skinny(A_codes, A_scales, a_format, B_codes, B_scales, bias, C, M, N, K, out_dtype, bias_dtype,
    #                        workspace, workspace_bytes, stream)
    assert lib.mase_gemm_mxfp4_skinny(p, p, 0, p, p, None, p, 4, 4, 192, 0, 0, p, 4096, None) == -2
    assert lib.mase_gemm_mxfp4_skinny(p, p, 0, p, p, None, p, 129, 4, 128, 0, 0, p, 4096, None) == -2
    assert lib.mase_gemm_mxfp4_skinny(p, None, 0, p, p, None, p, 4, 4, 128, 0, 0, p, 4096, None) == -1
    assert lib.mase_gemm_mxfp4_skinny(p, p, 2, p, p, None, p, 4, 4, 128, 0, 0, p, 4096, None) == -5   # activations: e4m3 or e5m2
    assert lib.mase_gemm_mxfp4_skinny(p, p, 0, p, p, None, p, 4, 4, 128, 7, 0, p, 4096, None) == -4
    assert lib.mase_gemm_mxfp4_skinny_workspace_bytes(4, 4, 192) == 0
    # mase_mxint_clip_search(in, ref, out, choice, numel, dtype, block_size, element_bits, scale_bits, tab, stream)
    assert lib.mase_mxint_clip_search(p, p, p, None, 64, 0, 8, 8, 8, p, None) == -5      # block sizes 16, 32, 64
    assert lib.mase_mxint_clip_search(p, p, p, None, 48, 0, 32, 8, 8, p, None) == -2
    assert lib.mase_mxint_clip_search(p, None, p, None, 64, 0, 32, 8, 8, p, None) == -1
    assert lib.mase_mxint_clip_search(p, p, p, None, 64, 0, 32, 1, 8, p, None) == -5
    assert lib.mase_mxint_clip_search(p, p, p, None, 64, 3, 32, 8, 8, p, None) == -4
    assert lib.mase_mxint_clip_search(p, p, p, None, 0, 0, 32, 8, 8, p, None) == 0
    assert lib.mase_mxfp_clip_search(p, p, p, None, 64, 0, 32, 3, 3, p, None) == -5      # illegal element format
    assert lib.mase_mxfp_clip_search(p, p, p, None, 64, 0, 128, 4, 3, p, None) == -5
    # mase_mxint_clip_candidates(in, cand, numel, dtype, block_size, element_bits, scale_bits, tab, stream)
    assert lib.mase_mxint_clip_candidates(p, p, 64, 0, 24, 8, 8, p, None) == -5
    assert lib.mase_mxint_clip_candidates(p, None, 64, 0, 32, 8, 8, p, None) == -1
    assert lib.mase_mxint_clip_candidates(p, p, 72, 0, 16, 8, 8, p, None) == -2
    assert lib.mase_mxint_clip_candidates(p, p, 0, 0, 16, 8, 8, p, None) == 0
    # mase_mxfp_clip_candidates(in, cand, score, numel, dtype, block_size, exp_bits, frac_bits, tab, stream)
    assert lib.mase_mxfp_clip_candidates(p, p, None, 64, 0, 32, 2, 1, p, None) == -1
    assert lib.mase_mxfp_clip_candidates(p, p, p, 64, 0, 32, 3, 3, p, None) == -5
    assert lib.mase_mxfp_clip_candidates(p, p, p, 64, 5, 32, 2, 1, p, None) == -4
    # mase_block_fp_qdq_static: the size limit is checked before anything touches a device
    assert lib.mase_block_fp_qdq_static(p, p, 1, 1, (1 << 20) + 1, 1, 1, 1, 8, 8, -1, 0, p, None) == -7
    assert lib.mase_block_fp_qdq_static(p, p, 0, 1, 16, 1, 16, 1, 8, 8, -1, 0, p, None) == 0
    assert lib.mase_mxfp_clip_search(p, p, None, None, 64, 0, 32, 4, 3, p, None) == -1
    assert lib.mase_mxfp_qdq(p, p, None, None, 64, 0, 0, 32, 3, 3, p, None) == -5  # illegal element format
    assert lib.mase_mxfp_qdq(p, p, None, None, 63, 0, 0, 32, 4, 3, p, None) == -2
    assert lib.mase_block_fp_qdq(p, p, 1, 4, 16, 0, 16, 0, 8, 8, -1, 0, p, None, 0, None) == -2
    assert lib.mase_block_fp_qdq(p, p, 1, 4, 16, 2, 16, 0, 8, 8, -1, 1, p, None, 0, None) == -7  # needs a workspace
    assert lib.mase_block_fp_qdq(p, p, 1, 4, 16, 1, 16, 2, 8, 2, 60, 0, p, None, 0, None) == -5  # 2^e underflows fp16
    assert lib.mase_integer_qdq(p, p, 16, 0, 40, 4, 1, 0, None) == -5
    assert lib.mase_minifloat_qdq(p, p, 16, 0, 8, 9, -1, 0, p, None) == -5
    assert lib.mase_minifloat_mx_qdq(p, p, 16, 0, 0, 4, 3, 1, 7, None) == -5
    assert lib.mase_block_fp_workspace_bytes(2, 5, 40, 2, 16, 1) == 2 * 3 * 3 * 4
    # packed-MXFP path: mase_mxfp_pack(in, codes, scales, numel, in_dtype, E, F, tab, stream)
    assert lib.mase_mxfp_pack(p, p, p, 48, 0, 4, 3, p, None) == -2       # whole blocks of 32
    assert lib.mase_mxfp_pack(p, p, p, 64, 0, 2, 3, p, None) == -5       # e2m3 has no matrix-instruction format
    assert lib.mase_mxfp_pack(p, None, p, 64, 0, 4, 3, p, None) == -1
    assert lib.mase_mxfp_pack(p, p, p, 64, 5, 4, 3, p, None) == -4
    # mase_gemm_mxfp_scaled(A, SA, a_fmt, B, SB, b_fmt, bias, C, M, N, K, out_dtype, bias_dtype, stream)
    assert lib.mase_gemm_mxfp_scaled(p, p, 0, p, p, 4, None, p, 4, 4, 192, 1, 0, None) == -2   # K in whole 128-tiles
    assert lib.mase_gemm_mxfp_scaled(p, p, 4, p, p, 4, None, p, 4, 4, 128, 1, 0, None) == -5   # A must be 8-bit
    assert lib.mase_gemm_mxfp_scaled(p, p, 0, p, p, 2, None, p, 4, 4, 128, 1, 0, None) == -5   # fp6 not provided
    assert lib.mase_gemm_mxfp_scaled(p, None, 0, p, p, 4, None, p, 4, 4, 128, 1, 0, None) == -1
    assert lib.mase_gemm_mxfp_scaled(p, p, 0, p, p, 4, None, p, 4, 4, 128, 3, 0, None) == -4
    assert lib.mase_gemm_mxfp_scaled(p, p, 0, p, p, 4, None, p, 0, 4, 128, 1, 0, None) == 0    # empty output


@pytest.mark.parametrize("dtype,code", [(torch.float32, 0), (torch.bfloat16, 1), (torch.float16, 2)])
def test_host_scalar_conversions_match_torch(lib, dtype, code):
    for v in (127, 255, 2047, 4095, 32767, 65535, -128, -2048, 1e-8, 3.3):
        want = torch.tensor(float(v)).to(dtype).float().item()
        assert lib.mase_round_scalar_to_dtype(float(v), code) == want
    # clamp really does cast its bounds to the tensor dtype
    if dtype != torch.float32:
        assert torch.tensor([5000.0], dtype=dtype).clamp(0, 2047).float().item() == lib.mase_round_scalar_to_dtype(2047.0, code)
    # isclose(x, 0) threshold
    thr = np.array([lib.mase_isclose_zero_threshold_bits(code)], dtype=np.uint32).view(np.float32)[0]
    zero = torch.tensor([0.0], dtype=dtype)
    t = torch.tensor([thr], dtype=torch.float32).to(dtype)
    assert t.float().item() == thr
    assert bool(torch.isclose(t, zero)) or thr == 0.0
    bigger = (t.view(torch.int16 if dtype != torch.float32 else torch.int32) + 1).view(dtype)
    assert not bool(torch.isclose(bigger, zero))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_log2_tables_reproduce_the_library(dtype):
    """the kernels' table lookup, replayed in numpy, equals torch.log2().ceil()/.floor() on the host"""
    from mase_amd._tables import log2_table_cpu

    tab = log2_table_cpu(dtype).astype(np.int64)
    if dtype == torch.float32:
        rng = np.random.default_rng(0)
        bits = np.concatenate([rng.integers(1, 0x7F800000, size=400000), 
                               (np.arange(1, 255)[:, None] << 23 | np.arange(0, 300)[None, :]).reshape(-1),
                               (np.arange(1, 255)[:, None] << 23 | (0x7FFFFF - np.arange(0, 300)[None, :])).reshape(-1),
                               np.arange(1, 5000)]).astype(np.uint32)
        v = torch.from_numpy(bits.view(np.int32).copy()).view(torch.float32)
    else:
        top = 0x7F80 if dtype == torch.bfloat16 else 0x7C00
        v = torch.arange(1, top, dtype=torch.int32).to(torch.int16).view(dtype)
    lg = v.log2()
    want_c = lg.ceil().float().numpy().astype(np.int64)
    want_f = lg.floor().float().numpy().astype(np.int64)
    mant, exp = np.frexp(v.double().numpy())
    k = exp.astype(np.int64) - 1
    M = np.rint((mant * 2 - 1) * (1 << 23)).astype(np.int64)
    got_c = np.where(M == 0, k, np.where(M <= tab[k + 149], k, k + 1))
    got_f = np.where(M >= tab[288 + k + 149], k + 1, k)
    assert np.array_equal(got_c, want_c) and np.array_equal(got_f, want_f)
    # summary words: inside [lo, hi] no correction exists; the extreme thresholds bound every entry
    lo, hi, mx = tab[277], tab[278], tab[279]
    assert np.all(tab[lo:hi + 1] == 0) and tab[:277].max() == mx
    lo, hi, mn = tab[288 + 277], tab[288 + 278], tab[288 + 279]
    assert np.all(tab[288 + lo:288 + hi + 1] == 0x800000) and tab[288:288 + 277].min() == mn


def test_block_fp_geometry_follows_the_reference_dispatch():
    from mase_amd.quantizers._ops import block_fp_geometry as g

    assert g((8, 2048, 4096), [1, 16], True) == (8, 2048, 4096, 1, 16, True)
    assert g((8, 2048, 4096), [16], True) == (8, 2048, 4096, 2048, 16, True)   # -1 prepended: whole token dim
    assert g((64, 128), [16], True) == (1, 64, 128, 1, 16, False)
    assert g((64, 128), [16], False) == (1, 64, 128, 64, 16, True)
    assert g((64, 128), [4, 256], False) == (1, 64, 128, 4, 128, True)            # oversize -> full dim
    assert g((100,), [16], False) == (1, 1, 100, 1, 16, False)
    assert g((100,), 16, False) == (1, 1, 100, 1, 16, False)
    assert g((10,), [2, 3, 16], False) == (1, 1, 10, 1, 10, False)
    with pytest.raises(AssertionError):
        g((100,), [16], True)
    with pytest.raises(NotImplementedError):
        g((2, 3, 4), [16], False)
    with pytest.raises(RuntimeError):
        g((2, 3, 4, 5), [16], True)


def test_product_has_no_cpu_path():
    import mase_amd.quantizers as Q
    from mase_amd._lib import MaseAmdError

    x = torch.randn(4, 32)
    for call in (lambda: Q.mxint_quantizer(x, 32, 8), lambda: Q.mxfp_quantizer(x, 32, 4, 3),
                 lambda: Q.block_fp_quantizer(x, 8, 8, None, [16]), lambda: Q.integer_quantizer(x, 8, 4),
                 lambda: Q.minifloat_denorm_quantizer(x, 8, 4), lambda: Q.minifloat_ieee_quantizer(x, 8, 4),
                 lambda: Q.mxint_quantizer(x, 32, 8, quantile_search=True),
                 lambda: Q.mxfp_quantizer(x, 32, 4, 3, quantile_search=True)):
        with pytest.raises(MaseAmdError):
            call()
    with pytest.raises(MaseAmdError):  # the search scored on calibration outputs runs on the device as well
        Q.mxint_quantizer_sim(x, -1, Q.MXIntMeta(block_size=32, scale_bits=8, element_bits=8),
                              act_tensor=x.reshape(1, 4, 32), quantile_search=True)


def test_product_does_not_import_the_oracle():
    import subprocess
    import sys

    code = "import sys; import mase_amd.quantizers, mase_amd.quantized, mase_amd.passes; assert not any(m == 'oracle' or m.startswith('oracle.') for m in sys.modules), 'oracle imported'"
    subprocess.run([sys.executable, "-c", code], check=True, cwd=ROOT)
    for dirpath, _, files in os.walk(os.path.join(ROOT, "mase_amd")):
        for f in files:
            if f.endswith(".py"):
                assert not re.search(r"^\s*(from|import)\s+oracle\b", open(os.path.join(dirpath, f)).read(), flags=re.M), f


def test_packed_mxfp_weight_eligibility_and_decoder_layer_host_side():
    """host logic that needs no GPU: which weights may take the block-scaled matrix instruction, and the synthetic
    decoder layer's shape/flop bookkeeping (it runs on the CPU with plain nn.Linear)"""
    from mase_amd.quantized.functional.mx_linear import PackedMXFPWeight
    from mase_amd.workloads import DecoderLayer, DecoderLayerConfig

    w = torch.zeros(64, 256)
    assert not PackedMXFPWeight.eligible(w, 32, (2, 1))            # not on a GPU
    assert not PackedMXFPWeight().valid_for(w)
    cfg = DecoderLayerConfig(hidden_size=256, num_heads=2, head_dim=128, intermediate_size=512)
    layer = DecoderLayer(cfg, dtype=torch.bfloat16, seed=3)
    again = DecoderLayer(cfg, dtype=torch.bfloat16, seed=3)
    assert torch.equal(layer.down_proj.weight, again.down_proj.weight)
    x = torch.randn(2, 16, 256).bfloat16()
    with torch.no_grad():
        y = layer(x)
        # causal: the first 8 positions do not depend on the rest
        y8 = layer(x[:, :8])
    assert y.shape == x.shape and y.dtype == torch.bfloat16
    assert (y[:, :8].float() - y8.float()).abs().max() < 0.1
    assert DecoderLayer(DecoderLayerConfig(), dtype=torch.bfloat16, device="meta").linear_flops(16384) == pytest.approx(6.632e12, rel=1e-3)


def test_module_pass_swaps_llama_blocks_on_the_host():
    """the swap itself needs no device: classes named like the Llama modules are matched through their bases, the
    replacements get network.config and the original weights"""
    from types import SimpleNamespace

    from mase_amd.passes import quantize_module_transform_pass
    from mase_amd.quantized import LlamaMLPMXFP, LlamaRMSNormMinifloat, quantized_module_map

    assert {"llama_self_attention_mxint", "llama_self_attention_mxfp", "llama_mlp_mxint", "llama_mlp_mxfp",
            "llama_rms_norm_minifloat"} <= set(quantized_module_map)

    class LlamaMLP(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_proj = torch.nn.Linear(64, 96, bias=False)
            self.up_proj = torch.nn.Linear(64, 96, bias=False)
            self.down_proj = torch.nn.Linear(96, 64, bias=False)

    class MyMLP(LlamaMLP):  # a subclass still matches
        pass

    class LlamaRMSNorm(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.full((64,), 1.5))

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.config = SimpleNamespace(hidden_size=64, intermediate_size=96, rms_norm_eps=1e-5)
            self.mlp, self.norm, self.act = MyMLP(), LlamaRMSNorm(), torch.nn.GELU()

    net = Net()
    up = net.mlp.up_proj.weight.detach().clone()
    args = {"by": "name",
            "mlp": {"config": {"name": "mxfp", "data_in_exponent_width": 4, "data_in_frac_width": 3}},
            "norm": {"config": {"name": "minifloat", "bypass": True}}}
    net, _ = quantize_module_transform_pass(net, args)
    assert isinstance(net.mlp, LlamaMLPMXFP) and torch.equal(net.mlp.up_proj.weight, up)
    assert net.mlp.q_config == {"data_in_exponent_width": 4, "data_in_frac_width": 3}  # "name" popped, as by name does
    assert isinstance(net.norm, LlamaRMSNormMinifloat) and float(net.norm.weight[0]) == 1.5
    assert net.norm.variance_epsilon == 1e-5 and net.norm.x_quantizer is None
    with pytest.raises(ValueError):
        quantize_module_transform_pass(net, {"by": "name", "act": {"config": {"name": "mxint"}}})


def test_unpack_rejects_bad_arguments_without_a_gpu(lib):
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.cast(buf, ctypes.c_void_p)
    # mase_mx_unpack(codes, scales, out, numel, block_size, out_dtype, kind, p0, p1, stream)
    assert lib.mase_mx_unpack(p, p, p, 0, 32, 0, 0, 8, 0, None) == 0
    assert lib.mase_mx_unpack(None, p, p, 64, 32, 0, 0, 8, 0, None) == -1
    assert lib.mase_mx_unpack(p, p, p, 65, 32, 0, 0, 8, 0, None) == -2
    assert lib.mase_mx_unpack(p, p, p, 64, 32, 0, 0, 9, 0, None) == -5     # codes are one byte
    assert lib.mase_mx_unpack(p, p, p, 64, 32, 0, 1, 5, 3, None) == -5     # sign + 5 + 3 bits do not fit a byte
    assert lib.mase_mx_unpack(p, p, p, 64, 32, 0, 2, 8, 0, None) == -5     # unknown kind
    assert lib.mase_mx_unpack(p, p, p, 64, 32, 7, 0, 8, 0, None) == -4


def test_attention_probability_entry_point_rejects_bad_arguments_without_a_gpu(lib):
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.cast(buf, ctypes.c_void_p)
    # (scores, mask, out, batch, heads, q_len, kv_len, mask_row_stride, dtype, scaling, cast E, F, finite, round,
    #  mx_kind, p0, p1, tab_dtype, tab_f32, stream)
    call = lib.mase_attn_softmax_mx
    assert call(p, None, p, 0, 4, 8, 64, 0, 1, 0.125, 4, 3, 1, 0, 1, 8, 0, p, None, None) == 0       # empty
    assert call(None, None, p, 1, 4, 8, 64, 0, 1, 0.125, 4, 3, 1, 0, 1, 8, 0, p, None, None) == -1
    assert call(p, None, p, 1, 4, 8, 48, 0, 1, 0.125, 4, 3, 1, 0, 1, 8, 0, p, None, None) == -2      # whole blocks of 32
    assert call(p, None, p, 1, 4, 8, 16384, 0, 1, 0.125, 4, 3, 1, 0, 1, 8, 0, p, None, None) == -2   # row too long
    assert call(p, p, p, 1, 4, 8, 64, 32, 1, 0.125, 4, 3, 1, 0, 1, 8, 0, p, None, None) == -2        # mask rows overlap
    assert call(p, None, p, 1, 4, 8, 64, 0, 5, 0.125, 4, 3, 1, 0, 1, 8, 0, p, None, None) == -4
    assert call(p, None, p, 1, 4, 8, 64, 0, 1, 0.125, 9, 3, 1, 0, 1, 8, 0, p, None, None) == -5      # cast format
    assert call(p, None, p, 1, 4, 8, 64, 0, 1, 0.125, 4, 3, 1, 0, 2, 3, 3, None, p, None) == -5      # MXFP format
    assert call(p, None, p, 1, 4, 8, 64, 0, 1, 0.125, 4, 3, 1, 0, 1, 8, 0, None, None, None) == -1   # table missing
    assert call(p, None, p, 1, 4, 8, 64, 0, 1, 0.125, 4, 3, 1, 0, 3, 8, 0, p, p, None) == -5         # unknown kind


def test_layer_op_entry_points_reject_bad_arguments_without_a_gpu(lib):
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.cast(buf, ctypes.c_void_p)
    # mase_rmsnorm_minifloat(x, weight, out, rows, cols, dtype, eps, x cast E F fin rm, w cast E F fin rm, stream)
    r = lib.mase_rmsnorm_minifloat
    assert r(p, p, p, 0, 64, 1, 1e-6, 0, 0, 1, 0, 0, 0, 1, 0, None) == 0
    assert r(p, None, p, 4, 64, 1, 1e-6, 0, 0, 1, 0, 0, 0, 1, 0, None) == -1
    assert r(p, p, p, 4, 60, 1, 1e-6, 0, 0, 1, 0, 0, 0, 1, 0, None) == -2      # whole 16-byte vectors
    assert r(p, p, p, 4, 16384, 1, 1e-6, 0, 0, 1, 0, 0, 0, 1, 0, None) == -2   # row too long for the registers
    assert r(p, p, p, 4, 64, 4, 1e-6, 0, 0, 1, 0, 0, 0, 1, 0, None) == -4
    assert r(p, p, p, 4, 64, 1, 1e-6, 9, 3, 1, 0, 0, 0, 1, 0, None) == -5      # cast format
    assert r(p, p, p, 4, 64, 1, 1e-6, 4, 3, 1, 0, 4, 3, 1, 7, None) == -5      # rounding mode
    # mase_add_rmsnorm_mxint(x, residual, weight, sum_out, out, rows, cols, dtype, eps, element_bits, log2_tab, stream)
    ar = lib.mase_add_rmsnorm_mxint
    assert ar(p, p, p, p, p, 0, 64, 1, 1e-6, 8, p, None) == 0
    assert ar(p, None, p, p, p, 4, 64, 1, 1e-6, 8, p, None) == -1    # no residual
    assert ar(p, p, p, None, p, 4, 64, 1, 1e-6, 8, p, None) == -1    # nowhere to put the sum
    assert ar(p, p, p, p, p, 4, 48, 1, 1e-6, 8, p, None) == -2       # whole blocks of 32
    assert ar(p, p, p, p, p, 4, 64, 3, 1e-6, 8, p, None) == -4
    assert ar(p, p, p, p, p, 4, 64, 1, 1e-6, 1, p, None) == -5       # element width
    # mase_rope(x, cos, sin, out, B, H, T, D, xs_b, xs_h, xs_t, cs_b, cs_t, dtype, stream)
    ro = lib.mase_rope
    assert ro(p, p, p, p, 0, 2, 4, 64, 512, 64, 128, 0, 64, 1, None) == 0
    assert ro(p, p, None, p, 1, 2, 4, 64, 512, 64, 128, 0, 64, 1, None) == -1
    assert ro(p, p, p, p, 1, 2, 4, 40, 512, 64, 128, 0, 64, 1, None) == -2      # head_dim in whole 16-element halves
    assert ro(p, p, p, p, 1, 2, 4, 64, 512, 60, 128, 0, 64, 1, None) == -2      # strides in whole vectors
    assert ro(p, p, p, p, 1, 2, 4, 64, 512, 64, 128, 0, 64, 6, None) == -4
    # mase_silu_mul_minifloat(gate, up, out, numel, dtype, E, F, fin, rm, stream)
    s = lib.mase_silu_mul_minifloat
    assert s(p, p, p, 0, 1, 0, 0, 1, 0, None) == 0
    assert s(p, p, None, 64, 1, 0, 0, 1, 0, None) == -1
    assert s(p, p, p, 63, 1, 0, 0, 1, 0, None) == -2
    assert s(p, p, p, 64, 3, 0, 0, 1, 0, None) == -4
    assert s(p, p, p, 64, 1, 4, 12, 1, 0, None) == -5


def test_gptq_host_logic_with_a_toy_quantizer():
    """The parts of the GPTQ pass that run on any device, with a stand-in quantizer (round to a grid of 1/4): the
    Cholesky factor satisfies U^T U = (G + damping)^-1; with a diagonal Gram matrix the result is plain rounding; with
    correlated inputs the output error on the calibration inputs tr(E G E^T) is below plain rounding's; the blocked
    feed-forward equals the group-by-group one; a dead input column comes out as zeros; and projections that read one
    tensor share one Gram matrix, fed once per sample."""
    from torch import nn

    from mase_amd.passes import gptq as GP

    g = torch.Generator().manual_seed(11)
    grid = lambda w, cal=None: torch.round(w * 4) / 4
    x = torch.randn(512, 64, generator=g) @ (torch.randn(64, 64, generator=g) * 0.4 + torch.eye(64))
    x[:, 5] = 0.0
    gram = GP.InputGram()
    gram.update(x[:256].reshape(2, 128, 64))
    gram.update(x[256:])
    assert gram.rows_seen == 512
    G = (x.double().t() @ x.double()).float()
    assert float((gram.matrix - G).abs().max() / G.abs().max()) < 1e-5
    U, dead = GP.inverse_cholesky_upper(gram.matrix)
    assert dead.tolist() == [i == 5 for i in range(64)]
    Gd = G.double().clone()
    Gd[5, 5] = 1.0
    Gd += 0.01 * torch.diagonal(Gd).mean() * torch.eye(64, dtype=torch.float64)
    assert float(((U.double().t() @ U.double()) @ Gd - torch.eye(64, dtype=torch.float64)).abs().max()) < 1e-3
    assert bool((torch.tril(U, -1) == 0).all())

    w = torch.randn(24, 64, generator=g)
    loss = lambda q: float((((w - q).double() @ G.double()) * (w - q).double()).sum())
    q = GP.round_weight(w, gram.matrix, 8, grid)
    assert bool((q[:, 5] == 0).all())
    assert torch.equal(q * 4, torch.round(q * 4))              # on the quantizer's grid
    live = [0, 1, 2, 3, 4, 6, 7]
    assert torch.equal(q[:, live], grid(w[:, live]))           # the first group has seen no feed-forward
    assert loss(q) < 0.8 * loss(grid(w))
    q1 = GP.round_weight(w, gram.matrix, 8, grid, panel_groups=1)
    q8 = GP.round_weight(w, gram.matrix, 8, grid, panel_groups=8)
    assert float((q == q1).float().mean()) > 0.995 and float((q == q8).float().mean()) > 0.995
    diag = torch.diag(torch.rand(64, generator=g) + 0.5)
    assert torch.equal(GP.round_weight(w, diag, 8, grid), grid(w))   # uncorrelated inputs: nothing to feed forward

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.self_attn = nn.Module()
            self.mlp = nn.Module()
            for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
                setattr(self.self_attn, name, nn.Linear(16, 16, bias=False))
            self.mlp.gate_proj, self.mlp.up_proj, self.mlp.down_proj = (nn.Linear(16, 32, bias=False), nn.Linear(16, 32, bias=False),
                                                                        nn.Linear(32, 16, bias=False))
            self.other = nn.Linear(16, 16)  # not named in PROJECTION_GROUPS: left alone

        def forward(self, h):
            a = self.self_attn
            h = h + a.o_proj(a.q_proj(h) * torch.sigmoid(a.k_proj(h)) + a.v_proj(h))
            m = self.mlp
            return self.other(h + m.down_proj(torch.sigmoid(m.gate_proj(h)) * m.up_proj(h)))

    torch.manual_seed(3)
    blk = Block()
    before = {n: m.weight.detach().clone() for n, m in GP.linear_modules(blk).items()}
    xs = [torch.randn(1, 40, 16, generator=g) for _ in range(3)]
    fed = []
    real = GP.InputGram.update
    GP.InputGram.update = lambda self, t: (fed.append(tuple(t.shape)), real(self, t))[1]
    try:
        names = GP.round_decoder_layer(blk, lambda j: blk(xs[j]), 3, grid, 8)
    finally:
        GP.InputGram.update = real
    assert names == ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj", "mlp.gate_proj",
                     "mlp.up_proj", "mlp.down_proj"]
    assert len(fed) == 4 * 3   # four distinct input tensors per forward (q/k/v share one, gate/up share one) x 3 samples
    after = GP.linear_modules(blk)
    for n in names:
        assert not torch.equal(after[n].weight, before[n]) and torch.equal(after[n].weight * 4, torch.round(after[n].weight * 4)), n
    assert torch.equal(after["other"].weight, before["other"])
    with pytest.raises(ValueError):
        GP.group_quantizer("int8", {"weight_block_size": 32}, True)
