"""Quantized ``nn.Linear`` modules with the constructors, config keys and ``load_state_dict`` behaviour of the
reference's ``chop/nn/quantized/modules/linear.py`` (``_LinearBase`` :61-83, ``LinearInteger`` :100-126,
``LinearMinifloatDenorm/IEEE`` :129-173, ``LinearBlockFP`` :199-219, ``LinearMXFP`` :817-895, ``LinearMXInt``
:898-972), so that the quantize pass can instantiate them through ``quantized_module_map`` unchanged.
"""
from __future__ import annotations

import torch
from torch.nn import functional as F

from ...quantizers import _ops, mxfp_quantizer, mxint_quantizer
from ..functional.linear import (QuantizedParamCache, linearBlockFP, linearInteger, linearMinifloatDenorm,
                                 linearMinifloatIEEE)
from ..functional.mx_linear import (MXIntCodeImage, PackedMXFPWeight, PackedMXIntWeight, WeightCache, mx_linear,
                                    mxfp_linear_native, mxfp_native_layout, mxfp_native_pack, mxint_codes_apply,
                                    mxint_decode_applies, mxint_linear_codes, mxint_linear_decode)


class _LinearBase(torch.nn.Linear):
    def __init__(self, in_features: int, out_features: int, bias: bool = False, device=None, dtype=None) -> None:
        super().__init__(in_features, out_features, bias, device, dtype)
        self.bypass = False
        self.pruning_masks = None
        self._param_cache = QuantizedParamCache()

    def _cache_for(self, config):
        """The reference quantizes weight and bias on every forward, and so does this module unless
        ``config["cache_quantized_params"]`` (not a key of the reference, default False) is set: then the quantized
        parameters are kept between inference forwards while the parameters are the same tensors at the same
        version.  An edit made through ``weight.data`` is not seen by that test; ``invalidate_weight_cache()`` after
        such an edit."""
        return self._param_cache if config.get("cache_quantized_params", False) else None

    def invalidate_weight_cache(self):
        """Forget the cached quantized parameters (needed only after an in-place edit through ``weight.data`` with
        ``cache_quantized_params`` on)."""
        self._param_cache.invalidate()


class LinearInteger(_LinearBase):
    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None, config=None,
                 out_config=None, floor=None) -> None:
        super().__init__(in_features, out_features, bias, device, dtype)
        assert config is not None, "config is None!"
        if floor is not None:
            config["floor"] = floor
        self.config = config
        self.out_config = out_config
        self.bypass = config.get("bypass", False)

    def forward(self, x):
        if self.bypass:
            return F.linear(x, self.weight, self.bias)
        return linearInteger(x, self.weight, self.bias, self.config, self.out_config,
                             param_cache=self._cache_for(self.config))


class _ConfigLinear(_LinearBase):
    _functional = None

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None,
                 config=None) -> None:
        super().__init__(in_features, out_features, bias, device, dtype)
        assert config is not None, "config is None!"
        self.config = config
        self.bypass = config.get("bypass", False)

    def forward(self, x):
        if self.bypass:
            return F.linear(x, self.weight, self.bias)
        return type(self)._functional(x, self.weight, self.bias, self.config, param_cache=self._cache_for(self.config))


class LinearMinifloatDenorm(_ConfigLinear):
    _functional = staticmethod(linearMinifloatDenorm)


class LinearMinifloatIEEE(_ConfigLinear):
    _functional = staticmethod(linearMinifloatIEEE)


class LinearBlockFP(_ConfigLinear):
    _functional = staticmethod(linearBlockFP)


class _LinearMX(_LinearBase):
    """Shared shape of LinearMXInt / LinearMXFP: weights (and optionally the bias) are quantized in place when a
    state dict is loaded; the forward quantizes the activations and contracts.  Inference only."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None,
                 config=None) -> None:
        super().__init__(in_features, out_features, bias, device, dtype)
        assert config is not None, "config is None!"
        self.config = config
        self.bypass = config.get("bypass", False)
        self.gptq = config.get("gptq", False)
        self.clip_search = config.get("clip_search", False)
        self._w_cache = WeightCache()

    def _quantize_params(self):
        raise NotImplementedError

    def invalidate_weight_cache(self):
        """Forget the bf16 image of the weight (needed only after an in-place edit through ``weight.data``)."""
        self._w_cache.invalidate()

    def load_state_dict(self, state_dict, strict=True, assign=False):
        """Load pretrained weights, then quantize them in place."""
        result = super().load_state_dict(state_dict, strict=strict, assign=assign)
        self._w_cache.invalidate()
        if self.bypass or self.gptq:
            return result
        self._before_quantize_params()
        self._quantize_params()
        self._after_quantize_params()
        return result

    def _before_quantize_params(self):
        pass

    def _after_quantize_params(self):
        pass

    def weights_loaded_quantized(self):
        """Tell the module that its parameters were just set to already quantized values (a packed checkpoint): the
        cached images are rebuilt from them on the next forward."""
        self._w_cache.invalidate()


class LinearMXInt(_LinearMX):
    """``config["packed_decode"]`` (default False; not a key of the reference) keeps the weight's MXINT8 codes and scale
    bytes next to the parameter (1.03 bytes per weight more) and lets forwards of at most 128 rows stream those instead
    of the bf16 image: the product of decode-sized batches is bound by the weight bytes, which this halves.  A packed
    checkpoint (``mase_amd.quantized.packed``) hands the codes over without this key.

    ``config["weight_memory"] = "codes"`` (default ``"bf16"``; not a key of the reference) makes forwards of more than
    128 rows run from the weight's MXINT8 codes as well: the tiled kernel takes them in fragment order (1.03 bytes per
    weight, built when the state dict is loaded) and widens them to bf16 in registers on the way into the matrix
    instruction, so neither the bf16 image of the weight nor its fragment-ordered copy (2 + 2 bytes per weight) is
    built.  Same results bit for bit; the contraction runs 10-16 % slower."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None,
                 config=None) -> None:
        super().__init__(in_features, out_features, bias, device, dtype, config)
        self._w_codes = PackedMXIntWeight()
        self._w_image = MXIntCodeImage()

    def invalidate_weight_cache(self):
        super().invalidate_weight_cache()
        self._w_codes.invalidate()
        self._w_image.invalidate()

    def _codes_mode(self) -> bool:
        return self.config.get("weight_memory", "bf16") == "codes"

    def weights_loaded_quantized(self, codes=None, scales=None):
        """``codes`` / ``scales``: the quantizer's codes and scale bytes of the weight when the caller has them (a packed
        checkpoint); kept for the decode path if they decode to exactly the weight."""
        super().weights_loaded_quantized()
        self._w_codes.invalidate()
        self._w_image.invalidate()
        if codes is None or self.bypass or self.gptq:
            return
        if not PackedMXIntWeight.eligible(self.weight, self.config["weight_block_size"], self.config["weight_width"]):
            return
        self._w_codes.set(codes.to(self.weight.device), scales.to(self.weight.device), self.weight)
        if not self._w_codes.decodes_to(self.weight.data):
            self._w_codes.invalidate()
        elif self._codes_mode() and MXIntCodeImage.eligible(self.weight, 32, 8):
            self._w_image.set(self._w_codes.codes, self._w_codes.scales, self.weight)

    def _quantize_params(self):
        cfg = self.config
        self._w_codes.invalidate()
        self._w_image.invalidate()
        want_image = self._codes_mode() and MXIntCodeImage.eligible(self.weight, cfg["weight_block_size"], cfg["weight_width"])
        want_codes = cfg.get("packed_decode", False) and PackedMXIntWeight.eligible(
            self.weight, cfg["weight_block_size"], cfg["weight_width"])
        if (want_image or want_codes) and not self.clip_search:
            deq, codes, scales = _ops.mxint_qdq(self.weight.data, 32, 8, 1, 8, pack=True)
            self.weight.data.copy_(deq)
            if want_codes:
                self._w_codes.set(codes, scales, self.weight)
            if want_image:
                self._w_image.set(codes, scales, self.weight)
        else:
            self.weight.data.copy_(
                mxint_quantizer(self.weight.data, block_size=cfg["weight_block_size"], element_bits=cfg["weight_width"],
                                block_dim=1, quantile_search=self.clip_search)
            )
        b_block_size = cfg.get("bias_block_size")
        b_element_bits = cfg.get("bias_width")
        if self.bias is not None and b_block_size is not None and b_element_bits is not None:
            self.bias.data.copy_(
                mxint_quantizer(self.bias.data, block_size=b_block_size, element_bits=b_element_bits, block_dim=0,
                                quantile_search=self.clip_search)
            )

    def _act_cfg(self):
        return self.config.get("data_in_block_size"), self.config.get("data_in_width")

    def activation_key(self, x):
        """what identifies this module's quantized form of ``x`` (``project_shared``); None when the forward does not
        go through the bf16 form of the quantized activations"""
        bs, bits = self._act_cfg()
        if (self.bypass or bs is None or bits is None or not x.is_cuda or x.numel() == 0
                or x.dtype not in (torch.float32, torch.bfloat16, torch.float16)):
            return None
        if (not mxint_decode_applies(x, self._w_codes, self.weight) and not mxint_codes_apply(x, self._w_image, self.weight)
                and self._w_cache.get(self.weight) is None):
            return None
        return ("mxint", bs, bits)

    def prepare_activation(self, x):
        bs, bits = self._act_cfg()
        return _ops.mxint_qdq(x.reshape(-1, x.shape[-1]), bs, bits, -1, 8, out_dtype=torch.bfloat16)

    @torch.no_grad()
    def forward(self, x, prepared=None):
        if self.bypass:
            return F.linear(x, self.weight, self.bias)
        bs, bits = self._act_cfg()
        if bs is None or bits is None:
            return F.linear(x, self.weight, self.bias)
        if mxint_decode_applies(x, self._w_codes, self.weight):
            return mxint_linear_decode(x, self._w_codes, self.bias, self.prepare_activation, xq=prepared)
        if mxint_codes_apply(x, self._w_image, self.weight):
            return mxint_linear_codes(x, self._w_image, self.bias, self.prepare_activation, xq=prepared)
        return mx_linear(
            x, self.weight, self.bias, self.prepare_activation,
            lambda t: mxint_quantizer(t, block_size=bs, element_bits=bits, block_dim=-1),
            self._w_cache, xq=prepared,
        )


class LinearMXFP(_LinearMX):
    """``config["native_mx"]`` (default True; not a key of the reference) lets the forward use the block-scaled
    matrix instruction when activations are e4m3/e5m2, weights e4m3/e5m2/e2m1, both block sizes are 32 and
    in_features is a multiple of 128; otherwise, or with ``native_mx=False``, the contraction runs in bf16 on the
    dequantized operands."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None,
                 config=None) -> None:
        super().__init__(in_features, out_features, bias, device, dtype, config)
        self._w_packed = PackedMXFPWeight()

    def invalidate_weight_cache(self):
        super().invalidate_weight_cache()
        self._w_packed.invalidate()

    def _weight_fmt(self):
        return (self.config["weight_exponent_width"], self.config["weight_frac_width"])

    def _before_quantize_params(self):
        self._w_packed.invalidate()
        if self.config.get("native_mx", True) and PackedMXFPWeight.eligible(
                self.weight, self.config["weight_block_size"], self._weight_fmt()):
            self._w_packed.pack(self.weight.data, self._weight_fmt())

    def _after_quantize_params(self):
        if self._w_packed.codes is not None:
            self._w_packed.bind(self.weight)

    def weights_loaded_quantized(self, codes=None, scales=None):
        """``codes`` / ``scales``: the quantizer's element codes and scale bytes of the weight, when the caller has
        them (a packed checkpoint).  The matrix-instruction image is built from them; it cannot be rebuilt from the
        quantized weight alone, because quantizing is not idempotent (an element equal to the smallest subnormal of
        the format quantizes to zero).  The image is kept only if it decodes to exactly the weight."""
        super().weights_loaded_quantized()
        self._w_packed.invalidate()
        if codes is None or self.bypass or self.gptq or not self.config.get("native_mx", True):
            return
        fmt = self._weight_fmt()
        if not PackedMXFPWeight.eligible(self.weight, self.config["weight_block_size"], fmt):
            return
        if self._w_packed.from_reference_codes(codes.to(self.weight.device), scales.to(self.weight.device), fmt) \
                and self._w_packed.decodes_to(self.weight.data):
            self._w_packed.bind(self.weight)
        else:
            self._w_packed.invalidate()

    def _quantize_params(self):
        cfg = self.config
        self.weight.data.copy_(
            mxfp_quantizer(self.weight.data, block_size=cfg["weight_block_size"],
                           element_exp_bits=cfg["weight_exponent_width"], element_frac_bits=cfg["weight_frac_width"],
                           block_dim=1)
        )
        b_block_size = cfg.get("bias_block_size")
        b_exp_bits = cfg.get("bias_exponent_width")
        b_frac_bits = cfg.get("bias_frac_width")
        if self.bias is not None and b_block_size is not None and b_exp_bits is not None:
            self.bias.data.copy_(
                mxfp_quantizer(self.bias.data, block_size=b_block_size, element_exp_bits=b_exp_bits,
                               element_frac_bits=b_frac_bits, block_dim=0)
            )

    def _act_cfg(self):
        return (self.config.get("data_in_block_size"), self.config.get("data_in_exponent_width"),
                self.config.get("data_in_frac_width"))

    def _native(self, x) -> bool:
        bs, eb, fb = self._act_cfg()
        return (bs == 32 and (eb, fb) in ((4, 3), (5, 2)) and x.is_cuda and x.dtype == self.weight.dtype
                and x.numel() > 0 and self._w_packed.valid_for(self.weight))

    def activation_key(self, x):
        """see ``LinearMXInt.activation_key``; the block-scaled path shares the packed codes, in the layout the
        contraction with this module's weight takes"""
        bs, eb, fb = self._act_cfg()
        if self.bypass or bs is None or eb is None or not x.is_cuda or x.numel() == 0:
            return None
        if self._native(x):
            return ("mxfp-codes", eb, fb, mxfp_native_layout(x, self._w_packed, (eb, fb)))
        if x.dtype not in (torch.float32, torch.bfloat16, torch.float16) or self._w_cache.get(self.weight) is None:
            return None
        return ("mxfp", bs, eb, fb)

    def prepare_activation(self, x):
        bs, eb, fb = self._act_cfg()
        if self._native(x):
            return mxfp_native_pack(x, (eb, fb), mxfp_native_layout(x, self._w_packed, (eb, fb)))
        return _ops.mxfp_qdq(x.reshape(-1, x.shape[-1]), bs, eb, fb, -1, 8, out_dtype=torch.bfloat16)

    @torch.no_grad()
    def forward(self, x, prepared=None):
        if self.bypass:
            return F.linear(x, self.weight, self.bias)
        bs, eb, fb = self._act_cfg()
        if bs is None or eb is None:
            return F.linear(x, self.weight, self.bias)
        if self._native(x):
            return mxfp_linear_native(x, self._w_packed, self.bias, (eb, fb), prepared=prepared)
        return mx_linear(
            x, self.weight, self.bias,
            lambda t: _ops.mxfp_qdq(t, bs, eb, fb, -1, 8, out_dtype=torch.bfloat16),
            lambda t: mxfp_quantizer(t, block_size=bs, element_exp_bits=eb, element_frac_bits=fb, block_dim=-1),
            self._w_cache, xq=prepared,
        )
