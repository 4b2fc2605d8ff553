"""ctypes binding of libmace_hip.so (the C ABI declared in include/mace_hip.h).

The library is the product; this module only loads it and declares argument types.  There
is no fallback: if the shared object is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmace_hip.so")

SUCCESS, INVALID_ARGS, OUT_OF_RESOURCES, UNSUPPORTED, RUNTIME_ERROR = range(5)
ROW_MAJOR, COL_MAJOR = 0, 1
REQUANT_REF, REQUANT_NEON = 0, 1
ACT_NOOP, ACT_RELU, ACT_RELUX = 0, 1, 2
MASK_NO_SMALL, MASK_NO_XRES, MASK_NO_MID, MASK_NO_XFLIP, MASK_NO_CONV_SHORT = 1, 2, 4, 8, 16
NOALLOC_SCRATCH_BYTES = 32 << 20

_STATUS_NAMES = {0: "MACE_SUCCESS", 1: "MACE_INVALID_ARGS", 2: "MACE_OUT_OF_RESOURCES",
                 3: "MACE_UNSUPPORTED", 4: "MACE_RUNTIME_ERROR"}

_i64, _i32, _f32, _int, _p = C.c_int64, C.c_int32, C.c_float, C.c_int, C.c_void_p

# name -> (restype, argtypes); must list every symbol of include/mace_hip.h
_GEMM_F32 = [_p, _p, _p, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _p]
_GEMV_F32 = [_p, _p, _p, _p, _i64, _i64, _i64, _int, _int, _p]
_GEMV_F32_ACT = [_p, _p, _p, _p, _i64, _i64, _i64, _int, _int, _int, _f32, _p]
_CONV_F32 = [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _int, _f32, _p]
_CONV2D_F32 = [_p, _p, _p, _p] + [_i64] * 7 + [_int] * 6 + [_int, _f32, _p]
_MATMUL_F32 = [_p, _p, _p, _p] + [_i64] * 5 + [_int] * 4 + [_p]
_GEMV_Q8_U8 = [_p, _p, _p, _p, _i64, _i64, _i64, _int, _int, _i32, _i32, _f32, _f32, _f32,
               _i32, _int, _p]
_GEMV_Q8_I32 = [_p, _p, _p, _p, _i64, _i64, _i64, _int, _int, _i32, _i32, _p]
_GEMM_Q8_I32 = [_p, _p, _int, _p, _int, _p, _int, _i64, _i64, _i64, _i64, _int, _int, _i32,
                _i32]
_GEMM_Q8_U8 = _GEMM_Q8_I32 + [_p, _i32, _int, _i32, _int, _int]
_CONV2D_Q8 = [_p, _p, _p, _p] + [_i64] * 7 + [_int] * 4 + [_f32, _i32, _f32, _i32, _f32, _f32, _i32,
                                                         _int, _int, _p]
_CONV_Q8 = [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _f32, _i32, _f32, _i32, _f32, _f32,
            _i32, _int, _int, _p]

SIGNATURES = {
    "mace_hip_ctx_create": (_int, [_int, C.POINTER(_p)]),
    "mace_hip_ctx_destroy": (_int, [_p]),
    "mace_hip_ctx_set_stream": (_int, [_p, _p]),
    "mace_hip_sync": (_int, [_p]),
    "mace_hip_last_error": (C.c_char_p, [_p]),
    "mace_hip_device_info": (_int, [_p, C.c_char_p, C.c_size_t, C.POINTER(_int),
                                    C.POINTER(_int)]),
    "mace_hip_timer_start": (_int, [_p]),
    "mace_hip_timer_stop": (_int, [_p, C.POINTER(_f32)]),
    "mace_hip_profile_enable": (_int, [_p, _int]),
    "mace_hip_profile_last_kernel_ms": (_int, [_p, C.POINTER(_f32)]),
    "mace_hip_profile_kernel_count": (_int, [_p, C.POINTER(_int)]),
    "mace_hip_profile_kernel_ms": (_int, [_p, _int, C.POINTER(_f32)]),
    "mace_hip_ctx_fail_next_allocs": (_int, [_p, _int]),
    "mace_hip_plan_ctx_create": (_int, [_int, _int, C.POINTER(_p)]),
    "mace_hip_last_plan": (_int, [_p, _p]),
    "mace_hip_plan_variant_count": (_int, [_int]),
    "mace_hip_plan_variant_valid": (_int, [_int, _int]),
    "mace_hip_plan_describe": (_int, [_int, _int, C.c_char_p, C.c_size_t]),
    "mace_hip_plan_coverage": (C.c_int64, [_int, _int]),
    "mace_hip_ctx_set_kernel_mask": (_int, [_p, _int]),
    "mace_hip_graph_capture_begin": (_int, [_p]),
    "mace_hip_graph_capture_end": (_int, [_p, C.POINTER(_p)]),
    "mace_hip_graph_launch": (_int, [_p, _p]),
    "mace_hip_graph_destroy": (_int, [_p, _p]),
    "mace_hip_malloc": (_int, [_p, C.c_size_t, C.POINTER(_p)]),
    "mace_hip_free": (_int, [_p, _p]),
    "mace_hip_memcpy_h2d": (_int, [_p, _p, _p, C.c_size_t]),
    "mace_hip_memcpy_d2h": (_int, [_p, _p, _p, C.c_size_t]),
    "mace_hip_weight_register": (_int, [_p, _p, C.c_size_t]),
    "mace_hip_weight_unregister": (_int, [_p, _p]),
    "mace_hip_host_weight_register": (_int, [_p, _p, C.c_size_t]),
    "mace_hip_host_weight_unregister": (_int, [_p, _p]),
    "mace_hip_host_weight_stats": (_int, [_p, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "mace_hip_weight_cache_stats": (_int, [_p, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "mace_hip_quantize_multiplier": (None, [C.c_double, C.POINTER(_i32), C.POINTER(_int)]),
    "mace_hip_get_output_multiplier_and_shift": (_int, [_f32, _f32, _f32, C.POINTER(_i32),
                                                        C.POINTER(_int)]),
    "mace_hip_quantize_u8": (C.c_uint8, [_f32, _f32, _i32]),
    "mace_hip_requant_fixed_u8": (C.c_uint8, [_i32, _i32, _int, _i32, _int, _int]),
    "mace_hip_adjust_range_u8": (None, [_f32, _f32, _int, C.POINTER(C.c_float), C.POINTER(C.c_int32)]),
    "mace_hip_find_min_max_f32": (_int, [_p, _p, _i64, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "mace_hip_quantize_tensor_u8": (_int, [_p, _p, _i64, _f32, _i32, _p]),
    "mace_hip_quantize_tensor_dynamic_u8": (_int, [_p, _p, _i64, _int, _p, C.POINTER(C.c_float), C.POINTER(C.c_int32)]),
    "mace_hip_dequantize_tensor_u8": (_int, [_p, _p, _i64, _f32, _i32, _p]),
    "mace_hip_dequantize_tensor_i32": (_int, [_p, _p, _i64, _f32, _i32, _p]),
    "mace_hip_quantize_tensor_u8_host": (_int, [_p, _p, _i64, _f32, _i32, _p]),
    "mace_hip_quantize_tensor_dynamic_u8_host": (_int, [_p, _p, _i64, _int, _p, C.POINTER(C.c_float), C.POINTER(C.c_int32)]),
    "mace_hip_dequantize_tensor_u8_host": (_int, [_p, _p, _i64, _f32, _i32, _p]),
    "mace_hip_dequantize_tensor_i32_host": (_int, [_p, _p, _i64, _f32, _i32, _p]),
    "mace_hip_requant_table_u8": (_int, [_i32, _i32, _int, _i32, _int, _int, C.POINTER(C.c_uint8)]),
    "mace_hip_requant_float_u8": (C.c_uint8, [_i32, _f32, _i32, _int]),
    "mace_hip_gemm_f32": (_int, _GEMM_F32),
    "mace_hip_gemm_f32_transpose": (_int, [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _int,
                                           _int, _int, _int, _int, _p]),
    "mace_hip_gemv_f32": (_int, _GEMV_F32),
    "mace_hip_gemv_f32_act": (_int, _GEMV_F32_ACT),
    "mace_hip_gemv_f32_act_host": (_int, _GEMV_F32_ACT),
    "mace_hip_conv1x1_f32_nchw": (_int, _CONV_F32),
    "mace_hip_conv2d_f32_nchw": (_int, _CONV2D_F32),
    "mace_hip_conv2d_f32_nchw_host": (_int, _CONV2D_F32),
    "mace_hip_matmul_f32": (_int, _MATMUL_F32),
    "mace_hip_matmul_f32_host": (_int, _MATMUL_F32),
    "mace_hip_gemv_q8_u8": (_int, _GEMV_Q8_U8),
    "mace_hip_gemv_q8_i32": (_int, _GEMV_Q8_I32),
    "mace_hip_gemm_q8_i32": (_int, _GEMM_Q8_I32),
    "mace_hip_gemm_q8_u8": (_int, _GEMM_Q8_U8),
    "mace_hip_gemm_q8_u8_noalloc": (_int, _GEMM_Q8_U8),
    "mace_hip_conv1x1_q8_nhwc": (_int, _CONV_Q8),
    "mace_hip_gemm_f32_host": (_int, _GEMM_F32),
    "mace_hip_gemv_f32_host": (_int, _GEMV_F32),
    "mace_hip_conv1x1_f32_nchw_host": (_int, _CONV_F32),
    "mace_hip_gemv_q8_u8_host": (_int, _GEMV_Q8_U8),
    "mace_hip_gemv_q8_i32_host": (_int, _GEMV_Q8_I32),
    "mace_hip_gemm_q8_i32_host": (_int, _GEMM_Q8_I32),
    "mace_hip_gemm_q8_u8_host": (_int, _GEMM_Q8_U8),
    "mace_hip_conv1x1_q8_nhwc_host": (_int, _CONV_Q8),
    "mace_hip_conv2d_q8_nhwc": (_int, _CONV2D_Q8),
    "mace_hip_conv2d_q8_nhwc_host": (_int, _CONV2D_Q8),
    "mace_hip_calc_padding_and_output_size": (_int, [_i64, _i64, _i64, _i64, _int, _int, _int, _int,
                                                     _int, C.POINTER(C.c_int64),
                                                     C.POINTER(C.c_int64), C.POINTER(_int),
                                                     C.POINTER(_int)]),
}


# kernel families (MACE_HIP_KF_*) and auxiliary passes (MACE_HIP_AUX_*) of include/mace_hip.h
(KF_NONE, KF_Q8_GEMM_FUSED_SMALL, KF_Q8_GEMM_XRES, KF_Q8_GEMM_MID, KF_Q8_GEMM_STREAM, KF_Q8_GEMM_RING,
 KF_Q8_GEMM_RING_XT, KF_Q8_GEMM_RING_XF, KF_Q8_GEMM_TILED, KF_Q8_GEMV_ROW, KF_Q8_GEMV_SLICE,
 KF_Q8_GEMV_MFMA_LDS, KF_Q8_GEMV_MFMA, KF_Q8_GEMV_ROWS, KF_Q8_GEMV_GENERAL, KF_F32_GEMM_VEC,
 KF_F32_GEMM_GENERAL, KF_F32_GEMM_FILL, KF_F32_GEMV_VEC, KF_F32_GEMV_GENERAL, KF_Q8_CONV_SHORT,
 KF_Q8_CONV_ROWS, KF_Q8_CONV_KSPLIT, KF_Q8_CONV_KSLICES, KF_COUNT) = range(25)
(AUX_PACK_ROWS, AUX_PACK_TRANSPOSE, AUX_PACK_SHIFTED, AUX_PANEL_SUMS, AUX_KMAJOR_SUMS, AUX_ZERO,
 AUX_IM2COL, AUX_BIAS_RESCALE, AUX_F32_PAD, AUX_FILL, AUX_WEIGHT_HIT, AUX_WEIGHT_BUILD,
 AUX_F32_KSPLIT, AUX_Q8_KSPLIT) = (1 << i for i in range(14))


class PlanStruct(C.Structure):
    _fields_ = [("family", _int), ("variant", _int), ("launches", _int), ("aux", _int),
                ("grid", _int * 3), ("block", _int), ("lds_bytes", _int)]


class Plan:
    """mace_hip_plan of a call: family / variant of its main kernel, launches, auxiliary passes."""

    def __init__(self, st):
        self.family, self.variant, self.launches, self.aux = st.family, st.variant, st.launches, st.aux
        self.grid, self.block, self.lds_bytes = tuple(st.grid), st.block, st.lds_bytes
        self.kernel = describe(self.family, self.variant)

    def __repr__(self):
        return "Plan(%s, launches=%d, aux=0x%x, grid=%s)" % (self.kernel, self.launches, self.aux,
                                                             self.grid)


def describe(family, variant):
    buf = C.create_string_buffer(256)
    if load().mace_hip_plan_describe(family, variant, buf, 256) != SUCCESS:
        raise ValueError("no kernel (family %d, variant %d)" % (family, variant))
    return buf.value.decode()


def variants(family):
    """Variant indices of a family that name an instantiation the library can launch."""
    lib = load()
    return [v for v in range(lib.mace_hip_plan_variant_count(family))
            if lib.mace_hip_plan_variant_valid(family, v)]


def coverage(family, variant):
    return load().mace_hip_plan_coverage(family, variant)


class MaceHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("%s: %s" % (_STATUS_NAMES.get(status, status), message))
        self.status = status


_lib = None


def load():
    """Load libmace_hip.so; raises if it has not been built (see __graft_entry__.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                "%s is missing: build it with `make -C mace_amd/csrc` "
                "(no CPU fallback exists)" % LIB_PATH)
        try:
            # PyTorch ships its own HIP runtime under the same soname; when both live in one
            # process the first one loaded is the one both use, and only PyTorch's request
            # resolves to a copy that is already there.  So let it go first when present.
            import torch  # noqa: F401
        except ImportError:
            pass
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)          # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class Context:
    """One stream + one scratch arena on one GPU (mace_hip_ctx)."""

    def __init__(self, device=0, plan_only=None):
        """plan_only=(cu_count, lds_bytes): a context that only plans (needs no GPU)."""
        self.lib = load()
        h = _p()
        if plan_only is not None:
            st = self.lib.mace_hip_plan_ctx_create(plan_only[0], plan_only[1], C.byref(h))
        else:
            st = self.lib.mace_hip_ctx_create(device, C.byref(h))
        if st != SUCCESS:
            raise MaceHipError(st, "mace_hip_ctx_create(device=%d) failed" % device)
        self.handle = h

    def last_plan(self):
        st = PlanStruct()
        self.check(self.lib.mace_hip_last_plan(self.handle, C.byref(st)))
        return Plan(st)

    def close(self):
        if getattr(self, "handle", None):
            self.lib.mace_hip_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def check(self, status):
        if status != SUCCESS:
            msg = self.lib.mace_hip_last_error(self.handle)
            raise MaceHipError(status, msg.decode() if msg else "")

    def call(self, name, *args):
        """Invoke a C entry point with this context as first argument, raising on error."""
        self.check(getattr(self.lib, name)(self.handle, *args))

    def status(self, name, *args):
        """Invoke and return the raw status code (for error-path tests)."""
        return getattr(self.lib, name)(self.handle, *args)

    def last_error(self):
        return self.lib.mace_hip_last_error(self.handle).decode()

    def sync(self):
        self.check(self.lib.mace_hip_sync(self.handle))

    def set_stream(self, stream_handle):
        self.check(self.lib.mace_hip_ctx_set_stream(self.handle, stream_handle))

    def device_info(self):
        buf = C.create_string_buffer(64)
        cu, lds = _int(), _int()
        self.check(self.lib.mace_hip_device_info(self.handle, buf, 64, C.byref(cu),
                                                 C.byref(lds)))
        return buf.value.decode(), cu.value, lds.value

    def timer_start(self):
        self.check(self.lib.mace_hip_timer_start(self.handle))

    def timer_stop(self):
        ms = _f32()
        self.check(self.lib.mace_hip_timer_stop(self.handle, C.byref(ms)))
        return ms.value


    def profile(self, on):
        self.check(self.lib.mace_hip_profile_enable(self.handle, int(on)))

    def last_kernel_ms(self):
        ms = _f32()
        self.check(self.lib.mace_hip_profile_last_kernel_ms(self.handle, C.byref(ms)))
        return ms.value

    def kernel_ms_list(self):
        """Durations of the launches timed since profile(True), oldest first (waits for them)."""
        n, ms = _int(), _f32()
        self.check(self.lib.mace_hip_profile_kernel_count(self.handle, C.byref(n)))
        out = []
        for i in range(max(0, n.value - 512), n.value):
            self.check(self.lib.mace_hip_profile_kernel_ms(self.handle, i, C.byref(ms)))
            out.append(ms.value)
        return out


def get_output_multiplier_and_shift(lhs_scale, rhs_scale, out_scale):
    m, s = _i32(), _int()
    st = load().mace_hip_get_output_multiplier_and_shift(lhs_scale, rhs_scale, out_scale,
                                                         C.byref(m), C.byref(s))
    if st != SUCCESS:
        raise MaceHipError(st, "output multiplier outside (0,1)")
    return m.value, s.value


def quantize_multiplier(multiplier):
    m, e = _i32(), _int()
    load().mace_hip_quantize_multiplier(multiplier, C.byref(m), C.byref(e))
    return m.value, e.value
