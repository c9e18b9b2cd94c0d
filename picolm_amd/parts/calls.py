"""The library's called operations (csrc/mixers.h) as a part emits them: each is a C function that
the engine hands the running step to, with a structure of sizes, offsets, constants and device
pointers.  The structures here mirror that header field by field."""
from __future__ import annotations

from ctypes import Structure, c_float, c_int32, c_int64, c_void_p

from .. import kernels


class LoopInputArgs(Structure):
    _fields_ = [("step", c_void_p), ("width", c_int32)]


class SinkAttentionArgs(Structure):
    _fields_ = [("n_heads", c_int32), ("n_kv_heads", c_int32), ("head_dim", c_int32), ("v_head_dim", c_int32),
                ("in_stride", c_int32), ("q_off", c_int32), ("k_off", c_int32), ("v_off", c_int32), ("gate_off", c_int32),
                ("scale", c_float), ("eps", c_float),
                ("q_norm", c_void_p), ("k_norm", c_void_p), ("bias", c_void_p), ("bias_rows", c_int32), ("sink", c_void_p), ("window", c_int32),
                ("chunk", c_int32), ("maps", c_int32), ("out_float", c_int32), ("unit_qk", c_int32), ("in_bias", c_void_p),
                ("cos_table", c_void_p), ("sin_table", c_void_p), ("table_positions", c_int32), ("rot_dims", c_int32), ("rot_half", c_int32)]


class ShortConvArgs(Structure):
    _fields_ = [("weight", c_void_p), ("bias", c_void_p), ("channels", c_int32), ("taps", c_int32),
                ("in_stride", c_int32), ("in_off", c_int32), ("out_stride", c_int32), ("out_off", c_int32),
                ("state_off", c_int64), ("act", c_int32)]


class StateScanArgs(Structure):
    _fields_ = [("rule", c_int32), ("n_heads", c_int32), ("n_key_heads", c_int32), ("key_dim", c_int32), ("value_dim", c_int32),
                ("in_stride", c_int32), ("a_off", c_int32), ("w_off", c_int32),
                ("qkv_stride", c_int32), ("q_off", c_int32), ("k_off", c_int32), ("v_off", c_int32),
                ("A_log", c_void_p), ("dt_bias", c_void_p), ("skip", c_void_p),
                ("unit_qk", c_int32), ("unit_eps", c_float), ("q_scale", c_float), ("state_off", c_int64)]


class GatedNormArgs(Structure):
    _fields_ = [("weight", c_void_p), ("weight_len", c_int32), ("width", c_int32), ("group", c_int32), ("eps", c_float),
                ("gate_first", c_int32), ("gate_stride", c_int32), ("gate_off", c_int32)]


class NormedSumArgs(Structure):
    _fields_ = [("w_a", c_void_p), ("w_b", c_void_p), ("width", c_int32), ("eps", c_float), ("mult", c_float)]


class MapRowsArgs(Structure):
    _fields_ = [("kind", c_int32), ("width", c_int32), ("in_dtype", c_int32), ("out_dtype", c_int32), ("param", c_float)]


class AddPositionsArgs(Structure):
    _fields_ = [("freq", c_void_p), ("width", c_int32)]


class TokenShiftArgs(Structure):
    _fields_ = [("mu", c_void_p), ("width", c_int32), ("state_off", c_int64)]


class GateRowsArgs(Structure):
    _fields_ = [("width", c_int32), ("act", c_int32), ("x_stride", c_int32), ("x_off", c_int32), ("x_dtype", c_int32),
                ("g_stride", c_int32), ("g_off", c_int32), ("out_dtype", c_int32), ("bias", c_void_p), ("g_per_row", c_int32)]


class SliceNormArgs(Structure):
    _fields_ = [("weight", c_void_p), ("width", c_int32), ("in_stride", c_int32), ("in_off", c_int32), ("out_stride", c_int32),
                ("out_off", c_int32), ("out_dtype", c_int32), ("eps", c_float)]


class HeadLinearArgs(Structure):
    _fields_ = [("weight", c_void_p), ("weight_dt", c_int32), ("heads", c_int32), ("in_dim", c_int32), ("out_dim", c_int32),
                ("transposed", c_int32), ("in_stride", c_int32), ("in_off", c_int32), ("in_dtype", c_int32),
                ("out_stride", c_int32), ("out_off", c_int32), ("out_dtype", c_int32),
                ("gate_act", c_int32), ("gate_stride", c_int32), ("gate_off", c_int32),
                ("in_head_stride", c_int32), ("out_head_stride", c_int32), ("gate_per_head", c_int32)]


class GatedPostnormArgs(Structure):
    _fields_ = [("weight", c_void_p), ("gate_bias", c_void_p), ("width", c_int32), ("alpha", c_float), ("eps", c_float)]


class ForgetGatesArgs(Structure):
    _fields_ = [("lower", c_void_p), ("bias", c_void_p), ("channels", c_int32), ("in_stride", c_int32), ("q_off", c_int32),
                ("f_off", c_int32)]


class DecayScanArgs(Structure):
    _fields_ = [("kind", c_int32), ("n_heads", c_int32), ("n_key_heads", c_int32), ("key_dim", c_int32), ("value_dim", c_int32),
                ("qk_stride", c_int32), ("q_off", c_int32), ("k_off", c_int32), ("a_off", c_int32),
                ("x_stride", c_int32), ("x_off", c_int32), ("dt_stride", c_int32), ("dt_off", c_int32),
                ("dt_bias", c_void_p), ("A", c_void_p), ("skip", c_void_p), ("state_off", c_int64)]


class RouteTopArgs(Structure):
    _fields_ = [("bias", c_void_p), ("experts", c_int32), ("top", c_int32), ("scoring", c_int32), ("in_stride", c_int32),
                ("scale", c_float)]


class RoutedExpertsArgs(Structure):
    _fields_ = [("gate", c_void_p), ("up", c_void_p), ("down", c_void_p), ("weight_dt", c_int32), ("experts", c_int32),
                ("top", c_int32), ("width", c_int32), ("ff", c_int32), ("adds", c_int32), ("identity", c_int32),
                ("act", c_int32), ("limit", c_float), ("alpha", c_float), ("weight_on_input", c_int32)]


class LayerNormArgs(Structure):
    _fields_ = [("weight", c_void_p), ("bias", c_void_p), ("width", c_int32), ("out_dtype", c_int32), ("eps", c_float),
                ("gathers", c_int32)]


class RotateHeadsArgs(Structure):
    _fields_ = [("cos_table", c_void_p), ("sin_table", c_void_p), ("table_positions", c_int32), ("dims", c_int32), ("half", c_int32),
                ("heads", c_int32), ("width", c_int32), ("in_stride", c_int32), ("in_off", c_int32), ("in_head_stride", c_int32),
                ("out_stride", c_int32), ("out_off", c_int32), ("out_head_stride", c_int32),
                ("more_heads", c_int32), ("more_in_off", c_int32), ("more_in_head_stride", c_int32), ("more_out_off", c_int32),
                ("more_out_head_stride", c_int32), ("norm_weight", c_void_p), ("norm_width", c_int32), ("norm_in_off", c_int32),
                ("norm_out_off", c_int32), ("norm_eps", c_float)]


class AddRowsArgs(Structure):
    _fields_ = [("vec", c_void_p), ("width", c_int32)]


class RmsPairArgs(Structure):
    _fields_ = [("w_a", c_void_p), ("w_b", c_void_p), ("width", c_int32), ("out_dtype", c_int32), ("eps", c_float)]


class MapDifferenceArgs(Structure):
    _fields_ = [("heads", c_int32), ("vdim", c_int32), ("out_dtype", c_int32), ("lam", c_float), ("eps", c_float), ("mult", c_float)]


GATE_NONE, GATE_SILU, GATE_SIGMOID = 0, 1, 2
DECAY_PER_ROW, DECAY_EXPONENTIAL = 1, 2
DECAY_SCAN_MAX_KEY_DIM = 256
MAP_RELU_SQUARED, MAP_SOFTCAP, MAP_SCALE = 1, 2, 3
SCORE_PICKED_SOFTMAX, SCORE_SOFTMAX_ALL, SCORE_SIGMOID = 0, 1, 2
EXPERT_SILU_GATED, EXPERT_CLAMPED = 0, 1
RULE_OUTER_PRODUCT, RULE_DELTA = 0, 1
STATE_SCAN_MAX_KEY_DIM = 256
SHORT_CONV_MAX_TAPS = 16


def emit_library_call(b, name: str, args: Structure, out: int, **kw) -> None:
    """Appends the library's operation `name` (`picolm_call_<name>`) with its arguments to the
    program; what it queues depends on device memory only."""
    b.call(getattr(kernels.lib(), "picolm_call_" + name), out=out, user=args, recordable=True, label=name, **kw)
