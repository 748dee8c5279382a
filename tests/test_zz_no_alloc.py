"""The entry point that allocates nothing, ``mase_block_fp_qdq_static``: same results as ``mase_block_fp_qdq`` with a
caller workspace, bit for bit, on two calls in a row (the second on a smaller input, so that what the first left in the
library's static scratch must not matter), for shapes that take the two-pass schedule (the one that uses the scratch);
the size limit is an error, not a fault."""
import pytest
import torch

from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu


def _call(lib, name, x, geom, width, ew, folded, tab, ws=None):
    from mase_amd import _lib

    batch, rows, cols, b0, b1 = geom
    out = torch.empty_like(x)
    args = [x.data_ptr(), out.data_ptr(), batch, rows, cols, b0, b1, _lib.dtype_code(x), width, ew, -1, int(folded),
            tab.data_ptr()]
    if ws is not None:
        args += [ws.data_ptr(), ws.numel() * 4]
    rc = getattr(lib, name)(*args, _lib.stream_ptr(x))
    return rc, out


def test_block_fp_static_matches_the_workspace_form_on_two_calls_in_a_row(dev):
    import oracle as O
    from mase_amd import _lib
    from mase_amd._tables import log2_table

    lib = _lib.load()
    g = torch.Generator().manual_seed(70)
    # (shape, block_size, skip_first_dim): tiles spanning rows, ragged edges, 3-D activations: all two-pass shapes;
    # the second of each pair is smaller than the first
    pairs = [(((6, 200, 328), [4, 24], True), ((3, 50, 72), [4, 24], True)),
             (((1024, 1000), [16, 16], False), ((96, 40), [16, 16], False)),
             (((2, 512, 1040), [1, 48], True), ((2, 100, 96), [1, 48], True))]
    for dtype in (torch.bfloat16, torch.float32, torch.float16):
        tab = log2_table(dtype, dev)
        for pair in pairs:
            for shape, block, skip in pair:          # the two calls in a row
                from mase_amd.quantizers._ops import block_fp_geometry

                x = (torch.randn(*shape, generator=g) * 3).to(dtype)
                x.view(-1)[::97] *= 40
                xd = x.to(dev)
                batch, rows, cols, b0, b1, folded = block_fp_geometry(shape, block, skip)
                geom = (batch, rows, cols, b0, b1)
                nws = lib.mase_block_fp_workspace_bytes(batch, rows, cols, b0, b1, _lib.dtype_code(xd)) // 4
                ws = torch.empty(nws, dtype=torch.int32, device=dev)
                rc_ws, want = _call(lib, "mase_block_fp_qdq", xd, geom, 8, 8, folded, tab, ws)
                rc_st, got = _call(lib, "mase_block_fp_qdq_static", xd, geom, 8, 8, folded, tab)
                assert rc_ws == 0 and rc_st == 0, (rc_ws, rc_st, shape, dtype)
                assert_bits_equal(got, want, f"static vs workspace {shape} {dtype}")
                ref = O.block_fp_quantizer(x.clone(), 8, 8, None, block, skip)
                assert_bits_equal(got, ref, f"static vs oracle {shape} {dtype}")
    # single-pass shapes go through the same entry point without touching the scratch
    x = torch.randn(4, 64, 256, generator=g).bfloat16().to(dev)
    tab = log2_table(torch.bfloat16, dev)
    rc, got = _call(lib, "mase_block_fp_qdq_static", x, (4, 64, 256, 1, 16), 8, 8, True, tab)
    rc2, want = _call(lib, "mase_block_fp_qdq", x, (4, 64, 256, 1, 16), 8, 8, True, tab, torch.empty(1, dtype=torch.int32, device=dev))
    assert rc == 0 and rc2 == 0
    assert_bits_equal(got, want, "single-pass shape")
    # beyond the static scratch: a clear error and no launch (2^20 + 1 tiles of one element each)
    n = _lib.BLOCK_FP_STATIC_MAX_TILES + 1
    big = torch.zeros(n, dtype=torch.bfloat16, device=dev)
    rc, _ = _call(lib, "mase_block_fp_qdq_static", big, (1, 1, n, 1, 1), 8, 8, False, tab)
    assert rc == -7 and lib.mase_error_string(rc).decode() == "workspace missing or too small"
    torch.cuda.synchronize()
