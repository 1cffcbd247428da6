"""ctypes binding of the C ABI declared in include/tsx_hip.h.

PyTorch is used only for device memory and streams: every function takes CUDA (HIP)
tensors, hands their raw pointers to libtsx_hip.so and returns tensors.  There is no CPU
fallback -- if the library is missing or a launch fails this module raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# TSX_HIP_LIBRARY overrides the in-tree library (e.g. a build kept elsewhere by the integrator).
LIB_PATH = os.environ.get("TSX_HIP_LIBRARY") or os.path.join(_HERE, "lib", "libtsx_hip.so")

_vp = ctypes.c_void_p
_i32 = ctypes.c_int32
_i64 = ctypes.c_int64
_f32 = ctypes.c_float
_sz = ctypes.c_size_t

ACT_NONE, ACT_RELU, ACT_LEAKY_RELU = 0, 1, 2
_ACT = {None: ACT_NONE, "none": ACT_NONE, "relu": ACT_RELU, "leaky_relu": ACT_LEAKY_RELU, "mish": 3, "mish_fast": 4}


class ConvGeom(ctypes.Structure):
    """tsx_conv2d_geom."""
    _fields_ = [(k, _i32) for k in ("n", "c", "h", "w", "cout", "kh", "kw", "pad_top", "pad_bottom", "pad_left",
                                    "pad_right", "stride_h", "stride_w", "dilation_h", "dilation_w")]


class Epilogue(ctypes.Structure):
    """tsx_epilogue."""
    _fields_ = [("dq_dev", _vp), ("row_scale_dev", _vp), ("bias_dev", _vp), ("act", _i32), ("slope", _f32),
                ("q_scales_dev", _vp), ("n_qscales", _i32), ("residual_dev", _vp), ("staged_out_dev", _vp),
                ("staged_hs", _i32), ("staged_ws", _i32), ("staged_cp", _i32), ("staged_pad_top", _i32),
                ("staged_pad_left", _i32), ("residual_after_act", _i32), ("staged_upsample", _i32)]


class TsxError(RuntimeError):
    pass


_lib = None

# name -> (restype, argtypes); every symbol include/tsx_hip.h declares.
SIGNATURES = {
    "tsx_last_error": (ctypes.c_char_p, []),
    "tsx_version": (ctypes.c_int, []),
    "tsx_device_cu_count": (ctypes.c_int, []),
    "tsx_conv2d_out_size": (ctypes.c_int, [ctypes.POINTER(ConvGeom), ctypes.POINTER(_i32), ctypes.POINTER(_i32)]),
    "tsx_quantize_f32_i8": (ctypes.c_int, [_vp, _i64, _vp, _i32, _vp, _vp]),
    "tsx_conv2d_i8_packed_weight_bytes": (_sz, [ctypes.POINTER(ConvGeom)]),
    "tsx_conv2d_i8_pack_weights": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, _vp]),
    "tsx_conv2d_i8_workspace_bytes": (_sz, [ctypes.POINTER(ConvGeom)]),
    "tsx_conv2d_i8_nchw": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, _f32, ctypes.POINTER(Epilogue), _vp, _vp,
                                          _vp, _vp, _sz, _vp]),
    "tsx_quantize_conv2d_i8_nchw": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, _i32, _vp, _f32,
                                                   ctypes.POINTER(Epilogue), _vp, _vp, _vp, _vp, _sz, _vp]),
    "tsx_noalloc_scratch_bytes": (_sz, []),
    "tsx_quantize_conv2d_i8_nchw_noalloc": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, _i32, _vp, _f32,
                                                           ctypes.POINTER(Epilogue), _vp, _vp, _vp, _vp]),
    "tsx_conv2d_i8_stage": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _i32, _vp, _i32, _f32, _vp, _sz, _vp]),
    "tsx_conv2d_i8_staged": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, ctypes.POINTER(Epilogue), _vp, _vp,
                                            _vp, _vp]),
    "tsx_conv2d_i8_staged_dims": (ctypes.c_int, [ctypes.POINTER(ConvGeom), ctypes.POINTER(_i32), ctypes.POINTER(_i32),
                                                 ctypes.POINTER(_i32)]),
    "tsx_conv2d_i8_stage_fill": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _f32, _vp, _sz, _vp]),
    "tsx_conv2d_i8_stage_fill_halo": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _f32, _vp, _sz, _vp]),
    "tsx_conv2d_i8_staged_at": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _i32, _i32, _vp, ctypes.POINTER(Epilogue), _vp,
                                               _vp, _vp, _vp]),
    "tsx_gemm_i8_packed_weight_bytes": (_sz, [_i32, _i32]),
    "tsx_gemm_i8_pack_weights": (ctypes.c_int, [_i32, _i32, _i32, _vp, _vp, _vp]),
    "tsx_gemm_i8_workspace_bytes": (_sz, [_i32, _i32]),
    "tsx_gemm_i8": (ctypes.c_int, [_i32, _i32, _i32, _vp, _vp, ctypes.POINTER(Epilogue), _vp, _vp, _vp, _vp, _sz, _vp]),
    "tsx_conv2d_f32_nchw": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, _f32, _vp, _i32, _f32, _vp, _vp]),
    "tsx_conv2d_f32_plan_info": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, ctypes.c_char_p, _sz]),
    "tsx_inner_prod_f32": (ctypes.c_int, [_i32, _i32, _i32, _vp, _vp, _i32, _vp, _vp]),
    "tsx_add_bias_f32": (ctypes.c_int, [_vp, _i64, _i32, _i64, _vp, _vp, _vp]),
    "tsx_relu_f32": (ctypes.c_int, [_vp, _i64, _vp, _vp]),
    "tsx_batch_norm_f32": (ctypes.c_int, [_vp, _i64, _i32, _i64, _vp, _vp, _f32, _vp, _vp]),
    "tsx_batch_scale_f32": (ctypes.c_int, [_vp, _i64, _i32, _i64, _vp, _vp, _vp, _vp]),
    "tsx_fused_batch_norm_f32": (ctypes.c_int, [_vp, _i64, _i32, _i64, _vp, _vp, _vp, _vp, _f32, _vp, _vp]),
    "tsx_leaky_relu_f32": (ctypes.c_int, [_vp, _i64, _f32, _vp, _vp]),
    "tsx_max_pooling2d_i8_staged": (ctypes.c_int, [_vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "tsx_add_f32": (ctypes.c_int, [_vp, _vp, _i64, _i32, _f32, _vp, _vp]),
    "tsx_add_broadcast_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32, _vp, _vp]),
    "tsx_mish_f32": (ctypes.c_int, [_vp, _i64, _vp, _vp]),
    "tsx_conv2d_i8_plan_info": (ctypes.c_int, [_vp, ctypes.c_char_p, _sz]),
    "tsx_softplus_f32": (ctypes.c_int, [_vp, _i64, _vp, _vp]),
    "tsx_tanh_f32": (ctypes.c_int, [_vp, _i64, _vp, _vp]),
    "tsx_mul_f32": (ctypes.c_int, [_vp, _vp, _i64, _vp, _vp]),
    "tsx_mul_broadcast_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32, _vp, _vp]),
    "tsx_concat_channels_f32": (ctypes.c_int, [_vp, _i64, _i32, _i64, _vp, _i32, _i32, _vp]),
    "tsx_resize_nearest_f32": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _i32, _i32, _vp]),
    "tsx_depthwise_conv2d_f32": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, _f32, _vp, _i32, _f32, _vp, _vp]),
    "tsx_pooling2d_out_size": (ctypes.c_int, [_i32] * 10 + [ctypes.POINTER(_i32), ctypes.POINTER(_i32)]),
    "tsx_pooling2d_f32": (ctypes.c_int, [_vp, _i64] + [_i32] * 10 + [_vp, _i32, _i32, _vp]),
    "tsx_winograd_f63_kernel_bytes": (_sz, [_i32, _i32]),
    "tsx_winograd_f63_transform_kernel": (ctypes.c_int, [_i32, _i32, _vp, _vp, _vp]),
    "tsx_winograd_f63_workspace_bytes": (_sz, [ctypes.POINTER(ConvGeom)]),
    "tsx_winograd_f23_kernel_bytes": (_sz, [_i32, _i32]),
    "tsx_winograd_f23_transform_kernel": (ctypes.c_int, [_i32, _i32, _vp, _vp, _vp]),
    "tsx_winograd_f23_workspace_bytes": (_sz, [ctypes.POINTER(ConvGeom)]),
    "tsx_conv2d_winograd_f23_nchw": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, _f32, _vp, _i32, _f32, _vp, _vp,
                                                    _sz, _vp]),
    "tsx_winograd_f63_fast_workspace_bytes": (_sz, [ctypes.POINTER(ConvGeom)]),
    "tsx_conv2d_winograd_f63_fast_nchw": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, _f32, _vp, _i32, _f32, _vp, _vp,
                                                         _sz, _vp]),
    "tsx_conv2d_winograd_f63_nchw": (ctypes.c_int, [ctypes.POINTER(ConvGeom), _vp, _vp, _f32, _vp, _i32, _f32, _vp, _vp,
                                                    _sz, _vp]),
}


def lib():
    """Load libtsx_hip.so (built in-tree by `python -m tennis_amd.build`); never falls back."""
    global _lib
    if _lib is None:
        # TSX_HIP_LIBRARY: another build of the same library (the measurement build with phase stamps and probes)
        path = os.environ.get("TSX_HIP_LIBRARY") or LIB_PATH
        if not os.path.exists(path):
            raise TsxError("%s is not built: run `python -m tennis_amd.build` (no CPU fallback exists)" % path)
        L = ctypes.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


AIDS_LIB_PATH = os.path.join(os.path.dirname(LIB_PATH), "libtsx_hip_aids.so")
_aids = None


def aids_lib():
    """The measurement build of the library (`python -m tennis_amd.build --aids`): the same entry points plus
    tsx_probe_mfma_i8 and tsx_debug_phase_stamps (csrc/tsx_aids.h), its kernels carrying phase stamps.  None where
    it is not built."""
    global _aids
    if _aids is None and os.path.exists(AIDS_LIB_PATH):
        L = ctypes.CDLL(AIDS_LIB_PATH)
        for name, (res, args) in list(SIGNATURES.items()) + [
                ("tsx_probe_mfma_i8", (ctypes.c_int, [_vp, _i32, _i32, _vp, _vp])),
                ("tsx_debug_phase_stamps", (ctypes.c_int, [_vp, _sz]))]:
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _aids = L
    return _aids


def check(rc):
    if rc != 0:
        raise TsxError("tsx error %d: %s" % (rc, lib().tsx_last_error().decode(errors="replace")))


def _ptr(t):
    return None if t is None else _vp(t.data_ptr())


def _stream():
    return _vp(torch.cuda.current_stream().cuda_stream)


def _dev(t, dtype):
    if t is None:
        return None
    if not t.is_cuda:
        raise TsxError("expected a device tensor")
    return t.to(dtype).contiguous() if (t.dtype != dtype or not t.is_contiguous()) else t


def make_geom(x_shape, w_shape, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1)):
    n, c, h, w = x_shape
    cout, cw, kh, kw = w_shape
    if cw != c:
        raise TsxError("weight channels %d != input channels %d" % (cw, c))
    return ConvGeom(n, c, h, w, cout, kh, kw, pads[0], pads[1], pads[2], pads[3], strides[0], strides[1],
                    dilations[0], dilations[1])


def conv_out_size(geom):
    ho, wo = _i32(), _i32()
    check(lib().tsx_conv2d_out_size(ctypes.byref(geom), ctypes.byref(ho), ctypes.byref(wo)))
    return ho.value, wo.value


def conv2d_i8_plan_info(geom):
    """tsx_conv2d_i8_plan_info: the kernels the plan of this layer launches, as a dict of its key=value words."""
    buf = ctypes.create_string_buffer(256)
    check(lib().tsx_conv2d_i8_plan_info(ctypes.byref(geom), buf, len(buf)))
    return dict(word.split("=", 1) for word in buf.value.decode().split())


def quantize(x, scales):
    """tsx_quantize_f32_i8: x fp32 device tensor, scales fp32 device tensor [x.shape[0]] (or [1])."""
    x = _dev(x, torch.float32)
    scales = _dev(scales, torch.float32)
    out = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    check(lib().tsx_quantize_f32_i8(_ptr(x), x.numel(), _ptr(scales), scales.numel(), _ptr(out), _stream()))
    return out


class _EpilogueArgs:
    """Keeps the device tensors of an epilogue alive next to the C struct."""

    def __init__(self, dq, bias=None, act=None, slope=0.0, q_scales=None, row_scale=None, residual=None, staged_out=None,
                 residual_after_act=False):
        self.dq = _dev(dq, torch.float32)
        self.bias = _dev(bias, torch.float32)
        self.q_scales = _dev(q_scales, torch.float32)
        self.row_scale = _dev(row_scale, torch.float32)
        self.residual = _dev(residual, torch.float32)
        self.c = Epilogue(_ptr(self.dq), _ptr(self.row_scale), _ptr(self.bias), _ACT[act], float(slope),
                          _ptr(self.q_scales), 0 if self.q_scales is None else self.q_scales.numel(),
                          _ptr(self.residual))
        self.c.residual_after_act = int(bool(residual_after_act))
        self.staged_out = staged_out     # StagedInput of the consuming convolution
        if staged_out is not None:
            self.c.staged_out_dev = staged_out.buf.data_ptr()
            self.c.staged_hs, self.c.staged_ws, self.c.staged_cp = staged_out.hs, staged_out.ws, staged_out.cp
            self.c.staged_pad_top, self.c.staged_pad_left = staged_out.pad_top, staged_out.pad_left
            self.c.staged_upsample = int(getattr(staged_out, "upsample", 1))


class StagedInput:
    """The staged (channel-blocked, padded) int8 input of one convolution for one input shape: producers write
    their requantized output straight into it, the convolution (and other consumers of the same tensor) read it."""

    def __init__(self, conv, x_shape, halo_only=False):
        """halo_only: the buffer starts as garbage and only what a producer does not write is set (what an
        operator whose output tensor is fresh memory on every run does)."""
        geom, _, ws_bytes = conv._plan(tuple(x_shape))
        hs, ws, cp = _i32(), _i32(), _i32()
        check(lib().tsx_conv2d_i8_staged_dims(ctypes.byref(geom), ctypes.byref(hs), ctypes.byref(ws), ctypes.byref(cp)))
        self.x_shape = tuple(x_shape)
        self.hs, self.ws, self.cp = hs.value, ws.value, cp.value
        self.pad_top, self.pad_left = conv.pads[0], conv.pads[2]
        self.buf = torch.full((max(ws_bytes, 16),), 0x55, dtype=torch.int8, device=conv.w.device)
        fill = lib().tsx_conv2d_i8_stage_fill_halo if halo_only else lib().tsx_conv2d_i8_stage_fill
        check(fill(ctypes.byref(geom), conv.padding_value, _ptr(self.buf), ws_bytes, _stream()))


class StagedPlain:
    """A staged int8 buffer without halo, [n][h][w][round_up(c, 64)], zero-initialised: a producer's requantized
    output in the pixel-major layout when the consumer is not a convolution (a pooling pass in between)."""

    def __init__(self, x_shape, device):
        n, c, h, w = x_shape
        self.x_shape = tuple(x_shape)
        self.hs, self.ws, self.cp = h, w, (c + 63) // 64 * 64
        self.pad_top = self.pad_left = 0
        self.buf = torch.zeros(n * h * w * self.cp, dtype=torch.int8, device=device)

    def column_pairs(self):
        """The same buffer as a map of half the width whose pixels are pairs of columns with twice the channels (for a
        producer that computes pairs of output columns: pair_outputs_weights)."""
        n, c, h, w = self.x_shape
        if c != self.cp or w % 2:
            raise TsxError("column pairs: %d channels in a pitch of %d, width %d" % (c, self.cp, w))
        v = object.__new__(StagedPlain)
        v.x_shape = (n, 2 * c, h, w // 2)
        v.hs, v.ws, v.cp = h, w // 2, 2 * self.cp
        v.pad_top = v.pad_left = 0
        v.buf = self.buf
        return v


class StagedSlice:
    """Channels [c0, c0 + channels) of a StagedInput, as the staged output of ONE producer of a channel concatenation:
    every producer's epilogue writes its requantized output into its own run of channels of the consumer's staged
    input (quantized with the consumer's scale, which was calibrated on the concatenated tensor), so the concatenated
    tensor never exists in fp32 and is never staged.  c0 must be a multiple of 16 (the epilogue stores 16 bytes)."""

    def __init__(self, staged, c0, channels, upsample=1):
        """upsample = 2: the producer's map is half the staged one's size and every pixel is written to the 2 x 2
        staged pixels it becomes under a nearest-neighbour resize (the epilogue's staged_upsample)."""
        n, c, h, w = staged.x_shape
        if c0 % 16 != 0 or c0 < 0 or c0 + channels > c:
            raise TsxError("channels [%d, %d) are not a 16-aligned run inside the %d of the staged tensor" % (c0, c0 + channels, c))
        if upsample not in (1, 2) or h % upsample or w % upsample:
            raise TsxError("staged slice: upsample %r does not fit a %dx%d map" % (upsample, h, w))
        self.upsample = upsample
        self.x_shape = (n, channels, h, w)
        self.hs, self.ws, self.cp = staged.hs, staged.ws, staged.cp
        self.pad_top, self.pad_left = staged.pad_top, staged.pad_left
        self.full_buf, self.c0 = staged.buf, c0
        self.buf = staged.buf[c0:]          # the epilogue takes the address of channel c0 of the first pixel


class StagedView:
    """Another consumer's view of a StagedInput that holds the same tensor with at least as much halo: the buffer
    entered `row0` rows and `col0` columns further in, with the owner's row and image pitch (what
    tsx_conv2d_i8_staged_at reads: a buffer whose extents are larger than the convolution needs)."""

    def __init__(self, owner, pad_top, pad_left):
        if pad_top > owner.pad_top or pad_left > owner.pad_left:
            raise TsxError("staged view: the owner's halo (%d, %d) is smaller than (%d, %d)" % (owner.pad_top, owner.pad_left, pad_top, pad_left))
        self.row0, self.col0 = owner.pad_top - pad_top, owner.pad_left - pad_left
        self.x_shape = owner.x_shape
        self.hs, self.ws, self.cp = owner.hs, owner.ws, owner.cp
        self.pad_top, self.pad_left = pad_top, pad_left
        self.full_buf = owner.buf
        self.buf = owner.buf[(self.row0 * owner.ws + self.col0) * owner.cp:]


class StagedPairs:
    """A StagedInput whose pixels are PAIRS of horizontally adjacent pixels of a tensor with half as many channels,
    seen as that tensor: the bytes of [hs][ws][cp] are those of [hs][2 ws][cp / 2].  A tensor of 32 channels staged
    by itself carries 32 bytes of padding per pixel; staged in pairs it carries none, and a 3 x 3 convolution of
    stride 2 over it is a 3 x 2 convolution of stride (2, 1) over the pairs (pair_columns_weights), with 6 K-steps
    instead of 9.  The producer's epilogue writes this view; the pair convolution reads `pairs`."""

    def __init__(self, staged):
        n, c2, h, w2 = staged.x_shape
        if c2 != staged.cp or c2 % 64:
            raise TsxError("staged pairs: %d channels per pair are not whole 64-channel blocks" % c2)
        self.pairs = staged
        self.x_shape = (n, c2 // 2, h, 2 * w2)
        self.hs, self.ws, self.cp = staged.hs, 2 * staged.ws, staged.cp // 2
        self.pad_top, self.pad_left = staged.pad_top, 2 * staged.pad_left
        self.buf = staged.buf


def pair_columns_weights(w):
    """Weights [cout][c][kh][3] of a convolution with column stride 2 and one column of left padding, rewritten for
    an input whose pixels are pairs of columns (channels [0, c): the even column, [c, 2c): the odd one):
    [cout][2c][kh][2] for column stride 1, one PAIR of left padding and none on the right.  Output column ow reads
    columns 2ow - 1 (odd half of pair ow - 1) and 2ow, 2ow + 1 (pair ow); the even half of pair ow - 1 gets zero
    weights, which add nothing to an integer sum: the accumulators are those of the original convolution."""
    cout, c, kh, kw = w.shape
    if kw != 3:
        raise TsxError("pair_columns_weights: kernel width %d, not 3" % kw)
    wp = torch.zeros((cout, 2 * c, kh, 2), dtype=w.dtype, device=w.device)
    wp[:, c:, :, 0] = w[:, :, :, 0]
    wp[:, :c, :, 1] = w[:, :, :, 1]
    wp[:, c:, :, 1] = w[:, :, :, 2]
    return wp


def pair_outputs_weights(w, stride_w=1):
    """Weights [cout][c][kh][kw] of a convolution with column stride stride_w, rewritten to produce PAIRS of output
    columns as one pixel of 2 cout channels: [2 cout][c][kh][kw + stride_w] for column stride 2 stride_w (same
    padding; an even number of output columns).  Channels [0, cout) are the even output column (kernel columns
    0..kw-1 of the wider window), [cout, 2 cout) the odd one (columns stride_w..stride_w+kw-1); the other columns carry
    zero weights.  Written as a staged hand-over this is byte for byte the layout of the unpaired map with cout
    channels per pixel; the dequantize scales and the bias are the original ones twice."""
    cout, c, kh, kw = w.shape
    wp = torch.zeros((2 * cout, c, kh, kw + stride_w), dtype=w.dtype, device=w.device)
    wp[:cout, :, :, :kw] = w
    wp[cout:, :, :, stride_w:] = w
    return wp


def staged_interior(staged, images):
    """The map inside a staged buffer (StagedInput / StagedPlain) as an int8 NCHW tensor of the given images:
    a copy, for checkers that compare a producer's requantized hand-over with the operator chain's values."""
    n, c, h, w = staged.x_shape
    c0 = getattr(staged, "c0", 0)
    buf = getattr(staged, "full_buf", staged.buf)
    t = buf[: n * staged.hs * staged.ws * staged.cp].view(n, staged.hs, staged.ws, staged.cp)
    top, left = staged.pad_top + getattr(staged, "row0", 0), staged.pad_left + getattr(staged, "col0", 0)
    t = t[list(images), top:top + h, left:left + w, c0:c0 + c]
    if getattr(staged, "upsample", 1) == 2:
        # the producer wrote every pixel four times: its own map is any of the four phases, and they must agree
        phases = [t[:, dy::2, dx::2] for dy in (0, 1) for dx in (0, 1)]
        if not all(torch.equal(phases[0], ph) for ph in phases[1:]):
            raise TsxError("staged slice: the 2 x 2 pixels of an upsampled hand-over differ")
        t = phases[0]
    return t.permute(0, 3, 1, 2).contiguous()


class Conv2dI8:
    """int8 conv2d with packed weights: the state a `conv2d_quantized` operator instance keeps.

    Mirrors base::Conv2DQuantized (src/backend/base/base_conv2d_quantized.cpp:13-219): the
    geometry and dequantize scales are fixed at init, weights are packed on first use.
    """

    def __init__(self, w_i8, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0):
        self.w = _dev(w_i8, torch.int8)
        self.pads, self.strides, self.dilations = tuple(pads), tuple(strides), tuple(dilations)
        self.padding_value = float(padding_value)
        self._packed = {}
        self._workspace = None

    def _plan(self, x_shape):
        geom = make_geom(x_shape, self.w.shape, self.pads, self.strides, self.dilations)
        key = (x_shape[1],)
        if key not in self._packed:
            nbytes = lib().tsx_conv2d_i8_packed_weight_bytes(ctypes.byref(geom))
            if nbytes == 0:
                raise TsxError("bad geometry: " + lib().tsx_last_error().decode())
            packed = torch.empty(nbytes, dtype=torch.uint8, device=self.w.device)
            check(lib().tsx_conv2d_i8_pack_weights(ctypes.byref(geom), _ptr(self.w), _ptr(packed), _stream()))
            self._packed[key] = packed
        ws_bytes = lib().tsx_conv2d_i8_workspace_bytes(ctypes.byref(geom))
        if self._workspace is None or self._workspace.numel() < ws_bytes:
            self._workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=self.w.device)
        return geom, self._packed[key], ws_bytes

    def stage(self, x, staged, x_scales=None):
        """Fill a StagedInput from an NCHW tensor: int8, or fp32 quantized with x_scales on the way."""
        fused_quant = x_scales is not None
        x = _dev(x, torch.float32 if fused_quant else torch.int8)
        geom, _, ws_bytes = self._plan(tuple(x.shape))
        xs = _dev(x_scales, torch.float32)
        check(lib().tsx_conv2d_i8_stage(ctypes.byref(geom), _ptr(x), int(fused_quant), _ptr(xs),
                                        0 if xs is None else xs.numel(), self.padding_value, _ptr(staged.buf), ws_bytes,
                                        _stream()))

    def run_staged(self, staged, dq, bias=None, act=None, slope=0.0, q_scales=None, want_f32=True, residual=None,
                   staged_out=None, residual_after_act=False):
        """The convolution on a StagedInput (its own, or another consumer's of the same tensor).  Returns
        (out_f32 or None, out_i8 or None); with staged_out the int8 output goes to that StagedInput instead."""
        geom, packed, _ = self._plan(staged.x_shape)
        ho, wo = conv_out_size(geom)
        shape = (staged.x_shape[0], self.w.shape[0], ho, wo)
        if residual is not None and tuple(residual.shape) != shape:
            raise TsxError("residual shape %s != output shape %s" % (tuple(residual.shape), shape))
        ep = _EpilogueArgs(dq, bias, act, slope, q_scales, residual=residual, staged_out=staged_out,
                           residual_after_act=residual_after_act)
        out_f32 = torch.empty(shape, dtype=torch.float32, device=self.w.device) if want_f32 else None
        out_i8 = (torch.empty(shape, dtype=torch.int8, device=self.w.device)
                  if (q_scales is not None and staged_out is None) else None)
        check(lib().tsx_conv2d_i8_staged_at(ctypes.byref(geom), _ptr(staged.buf), staged.hs, staged.ws, _ptr(packed),
                                            ctypes.byref(ep.c), _ptr(out_f32), _ptr(out_i8), None, _stream()))
        return out_f32, out_i8

    def __call__(self, x, dq=None, bias=None, act=None, slope=0.0, q_scales=None, x_scales=None,
                 want_f32=True, want_acc=False, residual=None, staged_out=None, residual_after_act=False):
        """x: int8 NCHW device tensor, or fp32 NCHW with x_scales (fused quantize); residual: fp32 tensor of
        the output's shape added before the activation.

        Returns (out_f32 or None, out_i8 or None, acc_i32 or None)."""
        fused_quant = x_scales is not None
        x = _dev(x, torch.float32 if fused_quant else torch.int8)
        geom, packed, ws_bytes = self._plan(tuple(x.shape))
        ho, wo = conv_out_size(geom)
        shape = (x.shape[0], self.w.shape[0], ho, wo)
        ep = (_EpilogueArgs(dq, bias, act, slope, q_scales, residual=residual, staged_out=staged_out,
                            residual_after_act=residual_after_act) if dq is not None else None)
        if residual is not None and tuple(residual.shape) != shape:
            raise TsxError("residual shape %s != output shape %s" % (tuple(residual.shape), shape))
        out_f32 = torch.empty(shape, dtype=torch.float32, device=x.device) if (want_f32 and ep) else None
        out_i8 = (torch.empty(shape, dtype=torch.int8, device=x.device)
                  if (ep and q_scales is not None and staged_out is None) else None)
        acc = torch.empty(shape, dtype=torch.int32, device=x.device) if want_acc else None
        epp = ctypes.byref(ep.c) if ep else None
        if fused_quant:
            xs = _dev(x_scales, torch.float32)
            check(lib().tsx_quantize_conv2d_i8_nchw(ctypes.byref(geom), _ptr(x), _ptr(xs), xs.numel(), _ptr(packed),
                                                    self.padding_value, epp, _ptr(out_f32), _ptr(out_i8), _ptr(acc),
                                                    _ptr(self._workspace), ws_bytes, _stream()))
        else:
            check(lib().tsx_conv2d_i8_nchw(ctypes.byref(geom), _ptr(x), _ptr(packed), self.padding_value, epp,
                                           _ptr(out_f32), _ptr(out_i8), _ptr(acc), _ptr(self._workspace), ws_bytes,
                                           _stream()))
        return out_f32, out_i8, acc


class GemmI8:
    """int8 GEMM (quantized inner_prod) with packed weights; rhs is [k][n], or [n][k] if transpose."""

    def __init__(self, w_i8, transpose=False):
        self.w = _dev(w_i8, torch.int8)
        self.transpose = bool(transpose)
        self.n, self.k = (self.w.shape if self.transpose else self.w.shape[::-1])
        nbytes = lib().tsx_gemm_i8_packed_weight_bytes(self.k, self.n)
        self.packed = torch.empty(nbytes, dtype=torch.uint8, device=self.w.device)
        check(lib().tsx_gemm_i8_pack_weights(self.k, self.n, int(self.transpose), _ptr(self.w), _ptr(self.packed),
                                             _stream()))
        self._workspace = None

    def __call__(self, a, dq=None, row_scale=None, bias=None, act=None, slope=0.0, q_scales=None, want_f32=True,
                 want_acc=False):
        a = _dev(a, torch.int8)
        m, k = a.shape
        if k != self.k:
            raise TsxError("lhs has %d columns, weights %d rows" % (k, self.k))
        ws_bytes = lib().tsx_gemm_i8_workspace_bytes(m, k)
        if a.data_ptr() % 16:
            ws_bytes = m * ((k + 63) // 64 * 64)
        if self._workspace is None or self._workspace.numel() < ws_bytes:
            self._workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=a.device)
        ep = _EpilogueArgs(dq, bias, act, slope, q_scales, row_scale) if dq is not None else None
        shape = (m, self.n)
        out_f32 = torch.empty(shape, dtype=torch.float32, device=a.device) if (want_f32 and ep) else None
        out_i8 = torch.empty(shape, dtype=torch.int8, device=a.device) if (ep and q_scales is not None) else None
        acc = torch.empty(shape, dtype=torch.int32, device=a.device) if want_acc else None
        check(lib().tsx_gemm_i8(m, self.n, k, _ptr(a), _ptr(self.packed), ctypes.byref(ep.c) if ep else None,
                                _ptr(out_f32), _ptr(out_i8), _ptr(acc), _ptr(self._workspace), ws_bytes, _stream()))
        return out_f32, out_i8, acc


def conv2d_f32(x, w, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0, bias=None, act=None,
               slope=0.0):
    """tsx_conv2d_f32_nchw: fp32 implicit-GEMM conv2d (optionally + add_bias + activation)."""
    x = _dev(x, torch.float32)
    w = _dev(w, torch.float32)
    bias = _dev(bias, torch.float32)
    geom = make_geom(tuple(x.shape), tuple(w.shape), pads, strides, dilations)
    ho, wo = conv_out_size(geom)
    out = torch.empty((x.shape[0], w.shape[0], ho, wo), dtype=torch.float32, device=x.device)
    check(lib().tsx_conv2d_f32_nchw(ctypes.byref(geom), _ptr(x), _ptr(w), float(padding_value), _ptr(bias), _ACT[act],
                                    float(slope), _ptr(out), _stream()))
    return out


def conv2d_f32_plan_info(x_shape, w, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1)):
    """tsx_conv2d_f32_plan_info as a dict ({"kernel": ..., "tiles": ...}) for an input of x_shape and weights w."""
    w = _dev(w, torch.float32)
    geom = make_geom(tuple(x_shape), tuple(w.shape), pads, strides, dilations)
    text = ctypes.create_string_buffer(256)
    check(lib().tsx_conv2d_f32_plan_info(ctypes.byref(geom), _ptr(w), text, 256))
    return dict(item.split("=", 1) for item in text.value.decode().split())


def conv2d_f32_prepared(x, w, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0, bias=None,
                        act=None, slope=0.0):
    """(launch, out): tsx_conv2d_f32_nchw on fixed tensors with every argument marshalled once, for callers that issue
    the same layer again and again (a layer of a few microseconds is otherwise bound by this module's per-call work:
    geometry, output allocation, argument conversion).  `launch()` enqueues one convolution on the stream that was
    current here and raises TsxError like conv2d_f32; `out` is the tensor it writes."""
    x = _dev(x, torch.float32)
    w = _dev(w, torch.float32)
    bias = _dev(bias, torch.float32)
    geom = make_geom(tuple(x.shape), tuple(w.shape), pads, strides, dilations)
    ho, wo = conv_out_size(geom)
    out = torch.empty((x.shape[0], w.shape[0], ho, wo), dtype=torch.float32, device=x.device)
    fn = lib().tsx_conv2d_f32_nchw
    args = (ctypes.byref(geom), _ptr(x), _ptr(w), float(padding_value), _ptr(bias), _ACT[act], float(slope), _ptr(out),
            _stream())
    keep = (x, w, bias, geom)

    def launch(_keep=keep):
        check(fn(*args))
    return launch, out


def inner_prod_f32(lhs, rhs, transpose=False):
    """tsx_inner_prod_f32: out[m][n] = lhs[m][k] * rhs ([k][n], or [n][k] when transpose)."""
    lhs = _dev(lhs, torch.float32)
    rhs = _dev(rhs, torch.float32)
    m, k = lhs.shape
    n = rhs.shape[0] if transpose else rhs.shape[1]
    if (rhs.shape[1] if transpose else rhs.shape[0]) != k:
        raise TsxError("inner_prod: inner extents differ")
    out = torch.empty((m, n), dtype=torch.float32, device=lhs.device)
    check(lib().tsx_inner_prod_f32(m, n, k, _ptr(lhs), _ptr(rhs), int(bool(transpose)), _ptr(out), _stream()))
    return out


class Winograd:
    """Winograd conv2d, mode "f63" or "f23": the state of a `conv2d_winograd` operator instance
    (transformed kernel cached at first use, base_conv2d_winograd.cpp:146-164)."""

    def __init__(self, w, pads=(0, 0, 0, 0), padding_value=0.0, mode="f63"):
        assert mode in ("f63", "f23")
        self.mode = mode
        self.w = _dev(w, torch.float32)
        self.pads = tuple(pads)
        self.padding_value = float(padding_value)
        cout, cin = self.w.shape[0], self.w.shape[1]
        L = lib()
        self._kernel_bytes = getattr(L, "tsx_winograd_%s_kernel_bytes" % mode)
        self._transform = getattr(L, "tsx_winograd_%s_transform_kernel" % mode)
        self._workspace_bytes = getattr(L, "tsx_winograd_%s_workspace_bytes" % mode)
        self._conv = getattr(L, "tsx_conv2d_winograd_%s_nchw" % mode)
        self.u = torch.empty(self._kernel_bytes(cout, cin) // 4, dtype=torch.float32, device=self.w.device)
        check(self._transform(cout, cin, _ptr(self.w), _ptr(self.u), _stream()))
        self._workspace = None

    def __call__(self, x, bias=None, act=None, slope=0.0, fast=False):
        """fast (f63 only): the MFMA form, held to the fp32 tolerance instead of the reference's bits."""
        x = _dev(x, torch.float32)
        bias = _dev(bias, torch.float32)
        geom = make_geom(tuple(x.shape), tuple(self.w.shape), self.pads)
        ho, wo = conv_out_size(geom)
        if fast:
            assert self.mode == "f63"
        nbytes = (lib().tsx_winograd_f63_fast_workspace_bytes if fast else self._workspace_bytes)(ctypes.byref(geom))
        if nbytes == 0:
            raise TsxError("winograd: " + lib().tsx_last_error().decode())
        if self._workspace is None or self._workspace.numel() < nbytes:
            self._workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        out = torch.empty((x.shape[0], self.w.shape[0], ho, wo), dtype=torch.float32, device=x.device)
        conv = lib().tsx_conv2d_winograd_f63_fast_nchw if fast else self._conv
        check(conv(ctypes.byref(geom), _ptr(x), _ptr(self.u), self.padding_value, _ptr(bias), _ACT[act],
                   float(slope), _ptr(out), _ptr(self._workspace), nbytes, _stream()))
        return out


class WinogradF63(Winograd):
    def __init__(self, w, pads=(0, 0, 0, 0), padding_value=0.0):
        super().__init__(w, pads, padding_value, "f63")


class WinogradF23(Winograd):
    def __init__(self, w, pads=(0, 0, 0, 0), padding_value=0.0):
        super().__init__(w, pads, padding_value, "f23")


def add_bias(x, bias, dim=1):
    x = _dev(x, torch.float32)
    bias = _dev(bias, torch.float32)
    pre = 1
    for d in x.shape[:dim]:
        pre *= d
    inner = 1
    for d in x.shape[dim + 1:]:
        inner *= d
    out = torch.empty_like(x)
    check(lib().tsx_add_bias_f32(_ptr(x), pre, x.shape[dim], inner, _ptr(bias), _ptr(out), _stream()))
    return out


def _channel_layout(x, dim):
    pre = 1
    for d in x.shape[:dim]:
        pre *= d
    inner = 1
    for d in x.shape[dim + 1:]:
        inner *= d
    return pre, x.shape[dim], inner


def batch_norm(x, mean, variance, epsilon=1e-5, dim=1):
    x = _dev(x, torch.float32)
    pre, ch, inner = _channel_layout(x, dim)
    out = torch.empty_like(x)
    check(lib().tsx_batch_norm_f32(_ptr(x), pre, ch, inner, _ptr(_dev(mean, torch.float32)), _ptr(_dev(variance, torch.float32)),
                                   float(epsilon), _ptr(out), _stream()))
    return out


def batch_scale(x, scale, bias, dim=1):
    x = _dev(x, torch.float32)
    pre, ch, inner = _channel_layout(x, dim)
    out = torch.empty_like(x)
    check(lib().tsx_batch_scale_f32(_ptr(x), pre, ch, inner, _ptr(_dev(scale, torch.float32)), _ptr(_dev(bias, torch.float32)),
                                    _ptr(out), _stream()))
    return out


def fused_batch_norm(x, mean, variance, scale, bias, epsilon=1e-5, dim=1):
    x = _dev(x, torch.float32)
    pre, ch, inner = _channel_layout(x, dim)
    out = torch.empty_like(x)
    check(lib().tsx_fused_batch_norm_f32(_ptr(x), pre, ch, inner, _ptr(_dev(mean, torch.float32)),
                                         _ptr(_dev(variance, torch.float32)), _ptr(_dev(scale, torch.float32)),
                                         _ptr(_dev(bias, torch.float32)), float(epsilon), _ptr(out), _stream()))
    return out


def relu(x):
    x = _dev(x, torch.float32)
    out = torch.empty_like(x)
    check(lib().tsx_relu_f32(_ptr(x), x.numel(), _ptr(out), _stream()))
    return out


def leaky_relu(x, scale):
    x = _dev(x, torch.float32)
    out = torch.empty_like(x)
    check(lib().tsx_leaky_relu_f32(_ptr(x), x.numel(), float(scale), _ptr(out), _stream()))
    return out


def add(a, b, act=None, slope=0.0, out=None):
    """tsx_add_f32: act(a + b) on equal shapes."""
    a = _dev(a, torch.float32)
    b = _dev(b, torch.float32)
    assert a.shape == b.shape
    if out is None:
        out = torch.empty_like(a)
    check(lib().tsx_add_f32(_ptr(a), _ptr(b), a.numel(), _ACT[act], float(slope), _ptr(out), _stream()))
    return out


def pool_out_size(h, w, ksize, pads, strides):
    oh, ow = _i32(), _i32()
    check(lib().tsx_pooling2d_out_size(h, w, ksize[0], ksize[1], pads[0], pads[1], pads[2], pads[3], strides[0],
                                       strides[1], ctypes.byref(oh), ctypes.byref(ow)))
    return oh.value, ow.value


def pooling2d(x, kind, ksize, strides, pads=(0, 0, 0, 0), white=False):
    """tsx_pooling2d_f32: kind "max" | "avg", pads = (top, bottom, left, right)."""
    x = _dev(x, torch.float32)
    n, c, h, w = x.shape
    ho, wo = pool_out_size(h, w, ksize, pads, strides)
    out = torch.empty((n, c, ho, wo), dtype=torch.float32, device=x.device)
    check(lib().tsx_pooling2d_f32(_ptr(x), n * c, h, w, {"max": 0, "avg": 1}[kind], pads[0], pads[2], ksize[0], ksize[1],
                                  strides[0], strides[1], int(white), _ptr(out), ho, wo, _stream()))
    return out


class StagedMap(ctypes.Structure):
    """tsx_staged_map."""
    _fields_ = [("data", ctypes.c_void_p), ("n", _i32), ("hs", _i32), ("ws", _i32), ("cp", _i32),
                ("pad_top", _i32), ("pad_left", _i32), ("h", _i32), ("w", _i32), ("c", _i32)]


def _staged_map(st):
    n, c, h, w = st.x_shape
    return StagedMap(_ptr(st.buf), n, st.hs, st.ws, st.cp, st.pad_top, st.pad_left, h, w, c)


def max_pooling2d_staged(src, dst, ksize, strides, pads=(0, 0, 0, 0)):
    """tsx_max_pooling2d_i8_staged between two StagedInput buffers (int8, pixel-major)."""
    ho, wo = pool_out_size(src.x_shape[2], src.x_shape[3], ksize, pads, strides)
    assert (ho, wo) == tuple(dst.x_shape[2:]), "destination map is not the pooled size"
    a, b = _staged_map(src), _staged_map(dst)
    check(lib().tsx_max_pooling2d_i8_staged(ctypes.byref(a), ctypes.byref(b), ksize[0], ksize[1], pads[0], pads[2],
                                            strides[0], strides[1], _stream()))
    return dst


def global_pooling2d(x, kind):
    return pooling2d(x, kind, tuple(x.shape[2:]), (1, 1))


def mish(x):
    x = _dev(x, torch.float32)
    out = torch.empty_like(x)
    check(lib().tsx_mish_f32(_ptr(x), x.numel(), _ptr(out), _stream()))
    return out


def softplus(x):
    x = _dev(x, torch.float32)
    out = torch.empty_like(x)
    check(lib().tsx_softplus_f32(_ptr(x), x.numel(), _ptr(out), _stream()))
    return out


def tanh(x):
    x = _dev(x, torch.float32)
    out = torch.empty_like(x)
    check(lib().tsx_tanh_f32(_ptr(x), x.numel(), _ptr(out), _stream()))
    return out


def mul(a, b):
    """tsx_mul_f32: a * b on equal shapes."""
    a, b = _dev(a, torch.float32), _dev(b, torch.float32)
    if a.shape != b.shape:
        raise TsxError("mul: shapes %s and %s differ" % (tuple(a.shape), tuple(b.shape)))
    out = torch.empty_like(a)
    check(lib().tsx_mul_f32(_ptr(a), _ptr(b), a.numel(), _ptr(out), _stream()))
    return out


def concat_channels(tensors):
    """cpu::Concat on dim 1 of NCHW tensors."""
    tensors = [_dev(t, torch.float32) for t in tensors]
    n, inner = tensors[0].shape[0], 1
    for d in tensors[0].shape[2:]:
        inner *= int(d)
    ctot = sum(t.shape[1] for t in tensors)
    out = torch.empty((n, ctot) + tuple(tensors[0].shape[2:]), dtype=torch.float32, device=tensors[0].device)
    off = 0
    for t in tensors:
        if t.shape[0] != n or tuple(t.shape[2:]) != tuple(tensors[0].shape[2:]):
            raise TsxError("concat: shapes differ outside dim 1")
        check(lib().tsx_concat_channels_f32(_ptr(t), n, t.shape[1], inner, _ptr(out), ctot, off, _stream()))
        off += t.shape[1]
    return out


def resize_nearest(x, ho, wo):
    x = _dev(x, torch.float32)
    n, c, h, w = x.shape
    out = torch.empty((n, c, ho, wo), dtype=torch.float32, device=x.device)
    check(lib().tsx_resize_nearest_f32(_ptr(x), n * c, h, w, _ptr(out), ho, wo, _stream()))
    return out


def depthwise_conv2d(x, w, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0, bias=None, act=None,
                     slope=0.0):
    """tsx_depthwise_conv2d_f32: w is [1, C, KH, KW]."""
    x = _dev(x, torch.float32)
    w = _dev(w, torch.float32)
    bias = _dev(bias, torch.float32)
    n, c, h, wd = x.shape
    geom = ConvGeom(n, c, h, wd, c, w.shape[2], w.shape[3], pads[0], pads[1], pads[2], pads[3], strides[0], strides[1],
                    dilations[0], dilations[1])
    ho, wo = conv_out_size(geom)
    out = torch.empty((n, c, ho, wo), dtype=torch.float32, device=x.device)
    check(lib().tsx_depthwise_conv2d_f32(ctypes.byref(geom), _ptr(x), _ptr(w), float(padding_value), _ptr(bias), _ACT[act],
                                         float(slope), _ptr(out), _stream()))
    return out
