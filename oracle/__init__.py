"""CPU oracle for the quantize-dequantize / quantized-Linear path.  TEST INFRASTRUCTURE ONLY.

This package restates, op for op with plain ``torch`` CPU calls, the arithmetic of the reference's
``chop.nn.quantizers`` functions and of the quantized ``Linear`` forward that consumes them.  It is the
checker the HIP kernels are compared against and the timed CPU baseline of the benchmark; nothing in
the shipped package ``mase_amd`` may import it.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` use it.

Why torch and not numpy/C: the reference's results depend on library behaviour of torch itself
(``Tensor.log2`` evaluated *in the tensor dtype*, ``pow(2, t)``, ``round`` half-to-even keeping the
sign of zero, bf16/fp16 ops computing in fp32 and rounding once, ``clamp`` casting its bounds to the
tensor dtype, ``isclose`` thresholds).  Restating those in another library would replace the very
behaviour that has to be matched.  Integer/bit arithmetic (`_minifloat_mx`) is additionally restated
as a scalar pure-integer routine in ``oracle/scalar.py`` so the two can be checked against each other.

Pinning status (what fixes each function besides reading the source):

* ``integer_quantizer``            closed form (exact rational arithmetic), exhaustive over bf16   -> pinned
* ``mxint_quantizer``              closed form with torch's own ``log2().ceil()``, invariants       -> pinned
* ``block_fp_quantizer``           blocking checked against a brute-force index map; element values: exact rational
                                   closed form in fp32; in bf16 / fp16 an op-by-op model with every rounding to the
                                   dtype written out (``oracle/scalar.py``: float64 arithmetic, where each single op is
                                   exact, plus an explicit round-to-fp32-then-dtype), and the closed form with the one
                                   rounding that matters; every finite 16-bit value as block maximum and as element,
                                   exponents from the library's own ``log2`` in the dtype               -> pinned
* ``minifloat_denorm/ieee``        exact closed form in fp32; in bf16 / fp16 the same explicit-rounding model over
                                   every finite 16-bit input for (8,4), (8,5), (6,3)                     -> pinned
* ``_minifloat_mx`` encode/decode  what the bit-field text computes, stated as a function of the input VALUE in exact
  and ``mxfp_quantizer``           arithmetic (carry out of the fraction: 2^(e+1) in even exponent fields, 2^e in odd
                                   ones; exponent field 0: truncation to the subnormal grid, zero for fraction 0;
                                   zero below 2^-bias; saturation; the 8-bit truncation before rounding), compared
                                   over every 16-bit high-half fp32 pattern, the same with non-zero low halves and a
                                   dense grid of ties, all six legal element formats x both ``is_finite`` x four
                                   rounding modes; plausible misreadings (ADD for the OR, rounded subnormals, rounding
                                   before truncation, gradual underflow) are each shown to fail that comparison
                                   (``tests/test_minifloat_mx_value_pins.py``); format invariants (codes fit 1+E+F
                                   bits, normal codes survive decode -> encode); the MXFP scale by exact arithmetic
                                                                                        -> pinned

* clip search (``quantile_search``)   quantile against exact rational interpolation; candidates against the scalar
                                   restatement; the choice against exact errors (first minimum, strict replace);
                                   the MXFP score against its formula on integer codes  -> pinned, except the
                                   library's summation order inside ``norm`` / ``sum`` and the uint8 power wrap,
                                   which are facts of the host library              -> parity unpinned (that part)

``tests/golden/known_answers.json`` holds small vectors computed with the exact scalar restatement (fp32 for all
quantizers, bf16 for block floating point in the headline configuration's format); the vectorised restatement (and
the kernels) must reproduce them bit for bit.

The reference ships no golden vectors or value-asserting tests for this path, and running the reference
to produce vectors was refused by the environment, so "parity unpinned" above means: restated from the
source text (file:line cited at each function), cross-checked by an independent scalar restatement, but
never compared with an execution of the reference.
"""
from .quantizers import (  # noqa: F401
    block_fp_quantizer,
    integer_floor_quantizer,
    integer_quantizer,
    minifloat_denorm_quantizer,
    minifloat_ieee_quantizer,
    minifloat_mx_compose,
    minifloat_mx_extract,
    minifloat_quantizer_sim,
    CLIP_PERCENTILES,
    mxfp_clip_search,
    mxfp_components,
    mxfp_quantizer,
    mxint_clip_search,
    mxint_components,
    mxint_quantizer,
)
from .linear import (  # noqa: F401
    linear_block_fp,
    linear_integer,
    linear_minifloat_denorm,
    linear_minifloat_ieee,
    linear_mxfp_forward,
    linear_mxint_forward,
)
