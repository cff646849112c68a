"""Python plumbing over libffk.so, the gfx950 operator-kernel library.

This module only loads the C-ABI library (``include/ffk.h``) with ctypes and
offers thin helpers that pass ``torch`` tensors' device pointers and the
current HIP stream to it.  PyTorch is used for device memory and streams only;
no arithmetic here is done by torch.  If ``libffk.so`` is missing the import of
any entry point fails loudly -- there is no fallback path.

The directory name contains a hyphen, so load it with
``importlib.util.spec_from_file_location('flexflow_train_amd', .../__init__.py)``
(see ``tests/conftest.py``).
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libffk.so")

c_int = ctypes.c_int
c_i64 = ctypes.c_int64
c_u64 = ctypes.c_uint64
c_f = ctypes.c_float
c_p = ctypes.c_void_p
c_sz = ctypes.c_size_t

# DataType ordinals of include/ffk.h
BOOL, INT32, INT64, HALF, FLOAT, DOUBLE, BF16 = range(7)
ERR_INVALID, ERR_HIP, ERR_UNSUPPORTED, ERR_WORKSPACE = 1, 2, 3, 4
ACT_NONE, ACT_RELU, ACT_SIGMOID, ACT_TANH, ACT_GELU = -1, 0, 1, 2, 3
AGGR_NONE, AGGR_SUM, AGGR_AVG = -1, 0, 1
OP = dict(
    SCALAR_MULTIPLY=8, SCALAR_ADD=9, SCALAR_TRUE_DIV=11, SCALAR_SUB=12, RELU=13,
    IDENTITY=14, SIGMOID=15, TANH=16, ELU=17, EW_ADD=28, EW_MUL=29, EW_SUB=35,
    EW_DIV=36, EW_MAX=40, EW_MIN=41, EXP=56, SIN=61, COS=62, GELU=67, RSQRT=70,
    POW=71, GELU_REFERENCE_GRAD=1067,
)


class FFKError(RuntimeError):
    """A non-zero status from the C ABI (the reference aborts in its place)."""


class AttentionDesc(ctypes.Structure):
    _fields_ = [
        ("batch", c_i64), ("heads", c_i64), ("seq_q", c_i64), ("seq_kv", c_i64),
        ("head_dim", c_i64),
        ("q_batch_stride", c_i64), ("q_seq_stride", c_i64),
        ("k_batch_stride", c_i64), ("k_seq_stride", c_i64),
        ("v_batch_stride", c_i64), ("v_seq_stride", c_i64),
        ("o_batch_stride", c_i64), ("o_seq_stride", c_i64),
        ("scale", c_f), ("causal", c_int),
        ("v_head_dim", c_i64),  # 0 = head_dim
    ]


class MHADesc(ctypes.Structure):
    _fields_ = [
        ("num_samples", c_i64), ("num_heads", c_i64),
        ("q_size", c_i64), ("k_size", c_i64), ("v_size", c_i64),
        ("q_proj_size", c_i64), ("k_proj_size", c_i64), ("v_proj_size", c_i64),
        ("o_proj_size", c_i64),
        ("qo_seq_length", c_i64), ("kv_seq_length", c_i64),
        ("scale", c_f), ("causal", c_int),
    ]


class EncoderLayerDesc(ctypes.Structure):
    _fields_ = [
        ("batch", c_i64), ("seq", c_i64), ("d_model", c_i64), ("heads", c_i64), ("d_ff", c_i64),
        ("dropout_rate", c_f), ("seed", c_u64), ("ln_eps", c_f), ("attn_scale", c_f),
        ("causal", c_int), ("pre_layer_norm", c_int), ("activation", c_int),
        ("overwrite_weight_grads", c_int),
    ]


class EncoderLayerParams(ctypes.Structure):
    _fields_ = [(n, c_p) for n in ("ln1_gamma", "ln1_beta", "attn_weight", "ln2_gamma", "ln2_beta",
                                   "w1", "b1", "w2", "b2")]


# name -> (restype, argtypes); must list every symbol include/ffk.h declares.
SIGNATURES = {
    "ffk_last_error": (ctypes.c_char_p, []),
    "ffk_device_count": (c_int, [ctypes.POINTER(c_int)]),
    "ffk_set_device": (c_int, [c_int]),
    "ffk_malloc": (c_int, [ctypes.POINTER(c_p), c_sz]),
    "ffk_free": (c_int, [c_p]),
    "ffk_host_malloc": (c_int, [ctypes.POINTER(c_p), c_sz]),
    "ffk_host_free": (c_int, [c_p]),
    "ffk_memcpy": (c_int, [c_p, c_p, c_sz, c_int, c_p]),
    "ffk_fill_zero": (c_int, [c_p, c_sz, c_p]),
    "ffk_stream_create": (c_int, [ctypes.POINTER(c_p)]),
    "ffk_stream_destroy": (c_int, [c_p]),
    "ffk_stream_synchronize": (c_int, [c_p]),
    "ffk_event_create": (c_int, [ctypes.POINTER(c_p)]),
    "ffk_event_destroy": (c_int, [c_p]),
    "ffk_event_record": (c_int, [c_p, c_p]),
    "ffk_event_synchronize": (c_int, [c_p]),
    "ffk_event_elapsed_ms": (c_int, [c_p, c_p, ctypes.POINTER(c_f)]),
    "ffk_probe_mfma_bf16": (c_int, [c_p, c_int, ctypes.c_uint32, c_p, c_sz, ctypes.POINTER(ctypes.c_double)]),
    "ffk_set_option": (c_int, [c_int, c_int]),
    "ffk_get_option": (c_int, [c_int, ctypes.POINTER(c_int)]),
    "ffk_linear_forward": (c_int, [c_p, c_int, c_int, c_p, c_p, c_p, c_p, c_i64, c_i64, c_i64]),
    "ffk_linear_backward_workspace_bytes": (c_sz, [c_int, c_int, c_int, c_i64, c_i64]),
    "ffk_linear_backward": (c_int, [c_p, c_int, c_int, c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p,
                                    c_i64, c_i64, c_i64, c_p, c_sz, c_int]),
    "ffk_linear_l2_regularizer_grad": (c_int, [c_p, c_int, c_p, c_p, c_i64, c_f]),
    "ffk_gemm": (c_int, [c_p, c_int, c_int, c_int, c_i64, c_i64, c_i64, c_p, c_p, c_p, c_int]),
    "ffk_gemm_kernel_name": (c_int, [c_int, c_int, c_int, c_i64, c_i64, c_i64, c_int, c_int, ctypes.c_char_p, c_sz]),
    "ffk_element_unary_forward": (c_int, [c_p, c_int, c_int, c_f, c_p, c_p, c_i64]),
    "ffk_element_unary_backward": (c_int, [c_p, c_int, c_int, c_f, c_p, c_p, c_p, c_p, c_i64,
                                           c_int]),
    "ffk_element_binary_forward": (c_int, [c_p, c_int, c_int, c_p, c_p, c_p, c_i64, c_i64,
                                           c_i64]),
    "ffk_element_binary_backward": (c_int, [c_p, c_int, c_int, c_p, c_p, c_p, c_p, c_p, c_i64,
                                            c_int]),
    "ffk_element_binary_backward_broadcast": (c_int, [c_p, c_int, c_int, c_p, c_p, c_p, c_p, c_p, c_i64,
                                                      c_i64, c_i64, c_int]),
    "ffk_layer_norm_forward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_i64, c_i64,
                                       c_f]),
    "ffk_layer_norm_backward_workspace_bytes": (c_sz, [c_i64, c_i64]),
    "ffk_layer_norm_backward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p,
                                        c_i64, c_i64, c_p, c_sz, c_int]),
    "ffk_layer_norm_backward_static": (c_int, [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p,
                                               c_p, c_i64, c_i64, c_int]),
    "ffk_dropout_backward_bias_grad_workspace_bytes": (c_sz, [c_i64, c_i64]),
    "ffk_dropout_backward_bias_grad": (c_int, [c_p, c_int, c_p, c_p, c_i64, c_i64, c_p, c_int, c_p, c_sz, c_f, c_u64,
                                               c_u64]),
    "ffk_linear_backward_dropout_gelu_bias_grad": (c_int, [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_i64, c_i64,
                                                           c_i64, c_p, c_sz, c_int, c_f, c_u64, c_u64, c_p, c_int, c_p,
                                                           c_sz]),
    "ffk_layer_norm_backward_residual": (c_int, [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p,
                                                 c_i64, c_i64, c_p, c_sz, c_int, c_p, c_f, c_u64, c_u64]),
    "ffk_dropout_add_layer_norm_forward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p,
                                                   c_i64, c_i64, c_f, c_f, c_u64, c_u64]),
    "ffk_softmax_forward": (c_int, [c_p, c_int, c_p, c_p, c_i64, c_i64, c_i64]),
    "ffk_softmax_backward_copy": (c_int, [c_p, c_int, c_p, c_p, c_sz]),
    "ffk_softmax_backward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_i64, c_i64, c_i64]),
    "ffk_dropout_forward": (c_int, [c_p, c_int, c_p, c_p, c_i64, c_f, c_u64, c_u64]),
    "ffk_dropout_backward": (c_int, [c_p, c_int, c_p, c_p, c_i64, c_f, c_u64, c_u64, c_int]),
    "ffk_dropout_mask": (c_int, [c_p, c_p, c_i64, c_f, c_u64, c_u64]),
    "ffk_column_reductions_begin": (c_int, []),
    "ffk_column_reductions_end": (c_int, [c_p]),
    "ffk_dropout_add_forward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_i64, c_f, c_u64, c_u64]),
    "ffk_gelu_dropout_forward": (c_int, [c_p, c_int, c_p, c_p, c_i64, c_f, c_u64, c_u64]),
    "ffk_dropout_gelu_backward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_i64, c_f, c_u64, c_u64]),
    "ffk_linear_gelu_dropout_forward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_i64, c_i64, c_i64, c_f,
                                                c_u64, c_u64]),
    "ffk_linear_dropout_add_forward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_i64, c_i64, c_i64, c_f,
                                               c_u64, c_u64]),
    "ffk_linear_backward_dropout_gelu": (c_int, [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_i64, c_i64,
                                                 c_i64, c_p, c_sz, c_int, c_f, c_u64, c_u64]),
    "ffk_sgd_update": (c_int, [c_p, c_int, c_f, c_f, c_int, c_f, c_p, c_i64, c_int, c_p, c_p, c_p]),
    "ffk_adam_update": (c_int, [c_p, c_int, c_f, c_f, c_f, c_f, c_f, c_p, c_i64, c_int, c_p, c_p,
                                c_p, c_p]),
    "ffk_sparse_categorical_crossentropy_loss_backward": (
        c_int, [c_p, c_p, c_p, c_p, c_i64, c_i64, c_int, c_int, c_int, c_f]),
    "ffk_categorical_crossentropy_loss_backward": (c_int, [c_p, c_p, c_p, c_p, c_i64, c_i64, c_f]),
    "ffk_mean_squared_error_avg_loss_backward": (c_int, [c_p, c_p, c_p, c_p, c_i64, c_i64, c_f]),
    "ffk_identity_loss_backward": (c_int, [c_p, c_p, c_p, c_i64, c_i64, c_f]),
    "ffk_cast_forward": (c_int, [c_p, c_int, c_int, c_p, c_p, c_i64]),
    "ffk_cast_backward": (c_int, [c_p, c_int, c_int, c_p, c_p, c_i64]),
    "ffk_transpose_forward": (c_int, [c_p, c_int, c_p, c_p, c_int, c_p, c_p]),
    "ffk_transpose_backward": (c_int, [c_p, c_int, c_p, c_p, c_int, c_p, c_p, c_int]),
    "ffk_gather_forward": (c_int, [c_p, c_int, c_int, c_p, c_p, c_p, c_i64, c_i64, c_i64, c_i64]),
    "ffk_gather_backward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_i64, c_i64, c_i64, c_i64]),
    "ffk_split_forward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_int, c_i64]),
    "ffk_split_backward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_int, c_i64, c_int]),
    "ffk_concat_forward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_int, c_i64]),
    "ffk_concat_backward": (c_int, [c_p, c_int, c_p, c_p, c_p, c_int, c_i64, c_int]),
    "ffk_embedding_forward": (c_int, [c_p, c_int, c_int, c_int, c_p, c_p, c_p, c_int, c_i64,
                                      c_i64, c_i64, c_i64]),
    "ffk_embedding_backward_workspace_bytes": (c_sz, [c_i64, c_i64]),
    "ffk_embedding_backward": (c_int, [c_p, c_int, c_int, c_p, c_p, c_p, c_int, c_i64, c_i64,
                                       c_i64, c_i64, c_int, c_p, c_sz]),
    "ffk_embedding_backward_typed": (c_int, [c_p, c_int, c_int, c_p, c_p, c_p, c_int, c_i64, c_i64, c_i64, c_i64]),
    "ffk_attention_forward": (c_int, [c_p, c_int, ctypes.POINTER(AttentionDesc), c_p, c_p, c_p,
                                      c_p, c_p]),
    "ffk_attention_backward": (c_int, [c_p, c_int, ctypes.POINTER(AttentionDesc), c_p, c_p, c_p,
                                       c_p, c_p, c_p, c_p, c_p, c_p, c_p]),
    "ffk_mha_weight_elements": (c_sz, [ctypes.POINTER(MHADesc)]),
    "ffk_mha_reserve_bytes": (c_sz, [ctypes.POINTER(MHADesc), c_int]),
    "ffk_mha_forward": (c_int, [c_p, c_int, ctypes.POINTER(MHADesc), c_p, c_p, c_p, c_p, c_p,
                                c_p, c_sz]),
    "ffk_mha_backward": (c_int, [c_p, c_int, ctypes.POINTER(MHADesc), c_p, c_p, c_p, c_p, c_p,
                                 c_p, c_p, c_p, c_p, c_p, c_sz, c_int]),
    "ffk_encoder_layer_workspace_bytes": (c_sz, [ctypes.POINTER(EncoderLayerDesc), c_int]),
    "ffk_encoder_layer_forward": (c_int, [c_p, c_int, ctypes.POINTER(EncoderLayerDesc),
                                          ctypes.POINTER(EncoderLayerParams), c_p, c_p, c_p, c_sz]),
    "ffk_encoder_layer_backward": (c_int, [c_p, c_int, ctypes.POINTER(EncoderLayerDesc),
                                           ctypes.POINTER(EncoderLayerParams),
                                           ctypes.POINTER(EncoderLayerParams), c_p, c_p, c_p, c_p,
                                           c_sz]),
}

_lib = None


def lib():
    """The loaded libffk.so with argtypes set; raises if it was never built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FFKError(
                "libffk.so is missing at %s: build it with "
                "`python flexflow-train_amd/build.py` (there is no fallback path)" % LIB_PATH
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


OPTION_GEMM_VARIANT, OPTION_LAYER_UNFUSED, OPTION_ATTENTION_VARIANT = 0, 1, 2


def set_option(which, value):
    """Process-wide tuning / test switch (see ffk_set_option in ffk.h)."""
    check(lib().ffk_set_option(which, int(value)))


def check(rc):
    if rc != 0:
        raise FFKError("ffk error %d: %s" % (rc, lib().ffk_last_error().decode()))


# --------------------------------------------------------------------------
# torch-tensor helpers
# --------------------------------------------------------------------------

def _torch():
    import torch
    return torch


def dtype_of(t):
    torch = _torch()
    table = {torch.float32: FLOAT, torch.bfloat16: BF16, torch.int32: INT32,
             torch.int64: INT64, torch.float16: HALF, torch.float64: DOUBLE,
             torch.bool: BOOL}
    return table[t.dtype]


def ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensor required"
    return t.data_ptr()


def current_stream():
    return _torch().cuda.current_stream().cuda_stream


def probe_mfma_bf16(iterations, out, seed=1):
    """Launches the matrix-rate probe on the current stream; returns the flops of the launch."""
    flops = ctypes.c_double()
    check(lib().ffk_probe_mfma_bf16(current_stream(), iterations, seed, ptr(out), out.numel() * out.element_size(),
                                    ctypes.byref(flops)))
    return flops.value


def linear_forward(x, w, b=None, activation=ACT_NONE, out=None):
    torch = _torch()
    batch, in_dim = x.shape
    out_dim = w.shape[0]
    if out is None:
        out = torch.empty((batch, out_dim), dtype=x.dtype, device=x.device)
    check(lib().ffk_linear_forward(current_stream(), dtype_of(x), activation, ptr(x), ptr(out),
                                   ptr(w), ptr(b), batch, in_dim, out_dim))
    return out


def linear_backward(y, dy, x, w, dx=None, dw=None, db=None, activation=ACT_NONE,
                    relu_grad_mode=0, accumulate=False, workspace=None):
    torch = _torch()
    batch, in_dim = x.shape
    out_dim = w.shape[0]
    if workspace is None:
        need = lib().ffk_linear_backward_workspace_bytes(dtype_of(x), activation,
                                                         int(db is not None), batch, out_dim)
        if need:
            workspace = torch.empty((need,), dtype=torch.uint8, device=x.device)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(lib().ffk_linear_backward(current_stream(), dtype_of(x), activation, relu_grad_mode,
                                    ptr(y), ptr(dy), ptr(x), ptr(dx), ptr(w), ptr(dw), ptr(db),
                                    batch, in_dim, out_dim, ptr(workspace), ws_bytes,
                                    7 if accumulate is True else int(accumulate)))
    return dx, dw, db


def gemm_kernel_name(dtype, trans_a, trans_b, M, N, K, has_bias=False, activation=ACT_NONE):
    """The kernel (template instance) the GEMM dispatch picks for a dense problem; launches nothing."""
    buf = ctypes.create_string_buffer(256)
    check(lib().ffk_gemm_kernel_name(dtype, int(trans_a), int(trans_b), M, N, K, int(has_bias), activation, buf, 256))
    return buf.value.decode()


def linear_l2_regularizer_grad(w, dw, lam):
    """dw = dw + lam * w in place (the L2 regulariser's term of Linear's weight gradient)."""
    check(lib().ffk_linear_l2_regularizer_grad(current_stream(), dtype_of(w), ptr(w), ptr(dw), w.numel(), lam))
    return dw


def linear_gelu_dropout_forward(x, w, b, rate, seed, offset=0):
    """(y, dropped): y = x . w^T + b, dropped = dropout(GELU(y)), one GEMM launch.
    Raises FFKError (FFK_ERR_UNSUPPORTED) for shapes without a fused kernel."""
    torch = _torch()
    batch, in_dim = x.shape
    out_dim = w.shape[0]
    y = torch.empty((batch, out_dim), dtype=x.dtype, device=x.device)
    dropped = torch.empty_like(y)
    check(lib().ffk_linear_gelu_dropout_forward(current_stream(), dtype_of(x), ptr(x), ptr(y), ptr(dropped),
                                                ptr(w), ptr(b), batch, in_dim, out_dim, rate, seed, offset))
    return y, dropped


def linear_dropout_add_forward(x, residual, w, b, rate, seed, offset=0):
    """residual + dropout(x . w^T + b), one GEMM launch."""
    torch = _torch()
    batch, in_dim = x.shape
    out_dim = w.shape[0]
    y = torch.empty((batch, out_dim), dtype=x.dtype, device=x.device)
    check(lib().ffk_linear_dropout_add_forward(current_stream(), dtype_of(x), ptr(x), ptr(residual), ptr(y),
                                               ptr(w), ptr(b), batch, in_dim, out_dim, rate, seed, offset))
    return y


def linear_backward_dropout_gelu(dy, x, gelu_input, w, rate, seed, offset=0, dw=None, db=None, accumulate=0):
    """Linear backward whose input gradient is dropout_backward(dy . w) * GELU'(gelu_input)."""
    torch = _torch()
    batch, in_dim = x.shape
    out_dim = w.shape[0]
    dx = torch.empty_like(x)
    need = lib().ffk_linear_backward_workspace_bytes(dtype_of(x), ACT_NONE, int(db is not None), batch, out_dim)
    workspace = torch.empty((max(need, 1),), dtype=torch.uint8, device=x.device)
    check(lib().ffk_linear_backward_dropout_gelu(current_stream(), dtype_of(x), ptr(dy), ptr(x), ptr(gelu_input),
                                                 ptr(dx), ptr(w), ptr(dw), ptr(db), batch, in_dim, out_dim,
                                                 ptr(workspace), need, int(accumulate), rate, seed, offset))
    return dx


def linear_backward_dropout_gelu_bias_grad(dy, x, gelu_input, w, rate, seed, gelu_bias_grad, offset=0, dw=None, db=None,
                                           accumulate=0, accumulate_gelu_bias=False):
    """linear_backward_dropout_gelu that also adds up the columns of the input gradient it writes."""
    torch = _torch()
    batch, in_dim = x.shape
    out_dim = w.shape[0]
    dx = torch.empty_like(x)
    need = lib().ffk_linear_backward_workspace_bytes(dtype_of(x), ACT_NONE, int(db is not None), batch, out_dim)
    workspace = torch.empty((max(need, 1),), dtype=torch.uint8, device=x.device)
    need2 = lib().ffk_dropout_backward_bias_grad_workspace_bytes(batch, in_dim)
    workspace2 = torch.empty((need2,), dtype=torch.uint8, device=x.device)
    check(lib().ffk_linear_backward_dropout_gelu_bias_grad(
        current_stream(), dtype_of(x), ptr(dy), ptr(x), ptr(gelu_input), ptr(dx), ptr(w), ptr(dw), ptr(db), batch,
        in_dim, out_dim, ptr(workspace), need, int(accumulate), rate, seed, offset, ptr(gelu_bias_grad),
        int(accumulate_gelu_bias), ptr(workspace2), need2))
    return dx


def dropout_backward_bias_grad(dy, rate, seed, bias_grad, offset=0, accumulate_bias=False):
    """dx = dropout_backward(dy) and bias_grad (+)= the column sums of dx, one pass."""
    torch = _torch()
    batch, out_dim = dy.shape
    dx = torch.empty_like(dy)
    need = lib().ffk_dropout_backward_bias_grad_workspace_bytes(batch, out_dim)
    workspace = torch.empty((need,), dtype=torch.uint8, device=dy.device)
    check(lib().ffk_dropout_backward_bias_grad(current_stream(), dtype_of(dy), ptr(dy), ptr(dx), batch, out_dim,
                                               ptr(bias_grad), int(accumulate_bias), ptr(workspace), need, rate, seed,
                                               offset))
    return dx


def gemm(A, B, C, trans_a=False, trans_b=False, accumulate=False):
    M, N = C.shape
    K = A.shape[0] if trans_a else A.shape[1]
    check(lib().ffk_gemm(current_stream(), dtype_of(A), int(trans_a), int(trans_b), M, N, K,
                         ptr(A), ptr(B), ptr(C), int(accumulate)))
    return C


def element_unary_forward(op, x, scalar=0.0, out=None):
    torch = _torch()
    if out is None:
        out = torch.empty_like(x)
    check(lib().ffk_element_unary_forward(current_stream(), dtype_of(x), op, scalar, ptr(x),
                                          ptr(out), x.numel()))
    return out


def element_unary_backward(op, y, dy, x, dx, scalar=0.0, accumulate=-1):
    check(lib().ffk_element_unary_backward(current_stream(), dtype_of(x), op, scalar, ptr(y),
                                           ptr(dy), ptr(x), ptr(dx), x.numel(), accumulate))
    return dx


def element_binary_forward(op, l, r, out=None):
    torch = _torch()
    if out is None:
        out = torch.empty_like(l if l.numel() >= r.numel() else r)
    check(lib().ffk_element_binary_forward(current_stream(), dtype_of(out), op, ptr(l), ptr(r),
                                           ptr(out), out.numel(), l.numel(), r.numel()))
    return out


def element_binary_backward(op, g, l, r, dl, dr, accumulate=False):
    check(lib().ffk_element_binary_backward(current_stream(), dtype_of(g), op, ptr(g), ptr(l),
                                            ptr(r), ptr(dl), ptr(dr), g.numel(),
                                            int(accumulate)))
    return dl, dr


def element_binary_backward_broadcast(op, g, l, r, dl, dr, accumulate=False):
    """Backward with operands that were broadcast over the leading dims; dl / dr may be None."""
    check(lib().ffk_element_binary_backward_broadcast(
        current_stream(), dtype_of(g), op, ptr(g), ptr(l), ptr(r), ptr(dl) if dl is not None else None,
        ptr(dr) if dr is not None else None, g.numel(), l.numel(), r.numel(), int(accumulate)))
    return dl, dr


def layer_norm_forward(x, gamma, beta, eps, out=None, mean=None, rstd=None):
    torch = _torch()
    M, N = x.shape
    if out is None:
        out = torch.empty_like(x)
    if mean is None:
        mean = torch.empty((M,), dtype=torch.float32, device=x.device)
    if rstd is None:
        rstd = torch.empty((M,), dtype=torch.float32, device=x.device)
    check(lib().ffk_layer_norm_forward(current_stream(), dtype_of(x), ptr(x), ptr(out),
                                       ptr(gamma), ptr(beta), ptr(mean), ptr(rstd), M, N, eps))
    return out, mean, rstd


# bits of ffk_layer_norm_backward's accumulate_input_grad
LN_ACC_INPUT, LN_ACC_PARAMS = 1, 2


def layer_norm_backward(dy, x, mean, rstd, gamma, dx, dgamma, dbeta, accumulate=False,
                        workspace=None):
    torch = _torch()
    M, N = x.shape
    need = lib().ffk_layer_norm_backward_workspace_bytes(M, N)
    if workspace is None:
        workspace = torch.empty((need,), dtype=torch.uint8, device=x.device)
    check(lib().ffk_layer_norm_backward(current_stream(), dtype_of(x), ptr(dy), ptr(x),
                                        ptr(mean), ptr(rstd), ptr(gamma), ptr(dx), ptr(dgamma),
                                        ptr(dbeta), M, N, ptr(workspace), workspace.numel(),
                                        int(accumulate)))
    return dx, dgamma, dbeta


def layer_norm_backward_static(dy, x, mean, rstd, gamma, dx, dgamma, dbeta, accumulate=False):
    """ffk_layer_norm_backward without a workspace: the library's own per-device array."""
    M, N = x.shape
    check(lib().ffk_layer_norm_backward_static(current_stream(), dtype_of(x), ptr(dy), ptr(x),
                                               ptr(mean), ptr(rstd), ptr(gamma), ptr(dx),
                                               ptr(dgamma), ptr(dbeta), M, N, int(accumulate)))
    return dx, dgamma, dbeta


def layer_norm_backward_residual(dy, x, mean, rstd, gamma, residual, dx, dgamma, dbeta, accumulate_params=False,
                                 dropped=None, rate=0.0, seed=0, offset=0, workspace=None):
    """dx = residual + LayerNorm gradient (one rounding); dropped (optional) = dropout_backward(dx)."""
    torch = _torch()
    M, N = x.shape
    if workspace is None:
        workspace = torch.empty((lib().ffk_layer_norm_backward_workspace_bytes(M, N),), dtype=torch.uint8,
                                device=x.device)
    check(lib().ffk_layer_norm_backward_residual(current_stream(), dtype_of(x), ptr(dy), ptr(x), ptr(mean), ptr(rstd),
                                                 ptr(gamma), ptr(residual), ptr(dx), ptr(dgamma), ptr(dbeta), M, N,
                                                 ptr(workspace), workspace.numel(), int(accumulate_params),
                                                 ptr(dropped), rate, seed, offset))
    return dx, dgamma, dbeta


def dropout_add_layer_norm_forward(x, residual, gamma, beta, eps, rate, seed, offset=0):
    """sum = residual + dropout(x); y = LayerNorm(sum).  Returns (sum, y, mean, rstd)."""
    torch = _torch()
    M, N = x.shape
    total, y = torch.empty_like(x), torch.empty_like(x)
    mean = torch.empty((M,), dtype=torch.float32, device=x.device)
    rstd = torch.empty((M,), dtype=torch.float32, device=x.device)
    check(lib().ffk_dropout_add_layer_norm_forward(current_stream(), dtype_of(x), ptr(x), ptr(residual), ptr(total),
                                                   ptr(y), ptr(gamma), ptr(beta), ptr(mean), ptr(rstd), M, N, eps,
                                                   rate, seed, offset))
    return total, y, mean, rstd


def softmax_forward(x, outer, dim, inner, out=None):
    torch = _torch()
    if out is None:
        out = torch.empty_like(x)
    check(lib().ffk_softmax_forward(current_stream(), dtype_of(x), ptr(x), ptr(out), outer, dim,
                                    inner))
    return out


def softmax_backward(y, dy, outer, dim, inner, dx=None):
    torch = _torch()
    if dx is None:
        dx = torch.empty_like(y)
    check(lib().ffk_softmax_backward(current_stream(), dtype_of(y), ptr(y), ptr(dy), ptr(dx),
                                     outer, dim, inner))
    return dx


def softmax_backward_copy(dy, dx=None):
    torch = _torch()
    if dx is None:
        dx = torch.empty_like(dy)
    check(lib().ffk_softmax_backward_copy(current_stream(), dtype_of(dy), ptr(dy), ptr(dx),
                                          dy.numel()))
    return dx


def dropout_forward(x, rate, seed, offset=0, out=None):
    torch = _torch()
    if out is None:
        out = torch.empty_like(x)
    check(lib().ffk_dropout_forward(current_stream(), dtype_of(x), ptr(x), ptr(out), x.numel(),
                                    rate, seed, offset))
    return out


def dropout_backward(dy, rate, seed, offset=0, dx=None, accumulate=False):
    torch = _torch()
    if dx is None:
        dx = torch.empty_like(dy)
    check(lib().ffk_dropout_backward(current_stream(), dtype_of(dy), ptr(dy), ptr(dx),
                                     dy.numel(), rate, seed, offset, int(accumulate)))
    return dx


def dropout_add_forward(x, residual, rate, seed, offset=0):
    """residual + dropout(x), one pass."""
    out = _torch().empty_like(x)
    check(lib().ffk_dropout_add_forward(current_stream(), dtype_of(x), ptr(x), ptr(residual), ptr(out), x.numel(),
                                        rate, seed, offset))
    return out


def gelu_dropout_forward(x, rate, seed, offset=0):
    """dropout(GELU(x)), one pass."""
    out = _torch().empty_like(x)
    check(lib().ffk_gelu_dropout_forward(current_stream(), dtype_of(x), ptr(x), ptr(out), x.numel(), rate, seed, offset))
    return out


def dropout_gelu_backward(dy, gelu_input, rate, seed, offset=0):
    """dropout_backward(dy) * GELU'(gelu_input), one pass."""
    dx = _torch().empty_like(dy)
    check(lib().ffk_dropout_gelu_backward(current_stream(), dtype_of(dy), ptr(dy), ptr(gelu_input), ptr(dx),
                                          dy.numel(), rate, seed, offset))
    return dx


def dropout_mask(n, rate, seed, offset=0, device="cuda"):
    torch = _torch()
    m = torch.empty((n,), dtype=torch.uint8, device=device)
    check(lib().ffk_dropout_mask(current_stream(), ptr(m), n, rate, seed, offset))
    return m


def sgd_update(weight, grad, lr, momentum=0.0, nesterov=False, weight_decay=0.0, sgd_v=None,
               num_replicas=1, weight_lowp=None):
    """In-place SGD step on fp32 `weight` (and `sgd_v`); grad is [num_replicas * n] fp32 or bf16."""
    n = weight.numel()
    check(lib().ffk_sgd_update(current_stream(), dtype_of(grad), lr, momentum, int(nesterov),
                               weight_decay, ptr(grad), n, num_replicas, ptr(weight), ptr(sgd_v),
                               ptr(weight_lowp)))
    return weight


def adam_update(weight, grad, adam_m, adam_v, alpha_t, beta1=0.9, beta2=0.999, weight_decay=0.0,
                epsilon=1e-8, num_replicas=1, weight_lowp=None):
    n = weight.numel()
    check(lib().ffk_adam_update(current_stream(), dtype_of(grad), alpha_t, beta1, beta2, weight_decay,
                                epsilon, ptr(grad), n, num_replicas, ptr(weight), ptr(adam_v),
                                ptr(adam_m), ptr(weight_lowp)))
    return weight


def sparse_categorical_crossentropy_loss_backward(logit, label, num_samples, num_classes, k,
                                                  scale_factor, out=None):
    torch = _torch()
    if out is None:
        out = torch.empty_like(logit)
    check(lib().ffk_sparse_categorical_crossentropy_loss_backward(
        current_stream(), ptr(out), ptr(logit), ptr(label), logit.numel(), out.numel(), num_samples,
        num_classes, k, scale_factor))
    return out


def difference_loss_backward(kind, logit, label, scale_factor, out=None):
    """kind: 'categorical_crossentropy' or 'mean_squared_error_avg'."""
    torch = _torch()
    if out is None:
        out = torch.empty_like(logit)
    fn = getattr(lib(), "ffk_%s_loss_backward" % kind)
    check(fn(current_stream(), ptr(out), ptr(logit), ptr(label), logit.numel(), out.numel(),
             scale_factor))
    return out


def identity_loss_backward(loss, scale_factor, out=None):
    torch = _torch()
    if out is None:
        out = torch.empty_like(loss)
    check(lib().ffk_identity_loss_backward(current_stream(), ptr(out), ptr(loss), loss.numel(),
                                           out.numel(), scale_factor))
    return out


def cast_forward(x, out):
    check(lib().ffk_cast_forward(current_stream(), dtype_of(x), dtype_of(out), ptr(x), ptr(out),
                                 x.numel()))
    return out


def cast_backward(out_grad, in_grad):
    check(lib().ffk_cast_backward(current_stream(), dtype_of(out_grad), dtype_of(in_grad),
                                  ptr(out_grad), ptr(in_grad), out_grad.numel()))
    return in_grad


def embedding_forward(indices, weight, aggr=AGGR_NONE, out_dtype=None):
    torch = _torch()
    V, D = weight.shape
    if aggr == AGGR_NONE:
        num_bags, bag = indices.numel(), 1
    else:
        bag = indices.shape[-1]
        num_bags = indices.numel() // bag
    out_dtype = out_dtype or weight.dtype
    out = torch.empty((num_bags, D), dtype=out_dtype, device=weight.device)
    check(lib().ffk_embedding_forward(current_stream(), dtype_of(indices), dtype_of(weight),
                                      dtype_of(out), ptr(indices), ptr(out), ptr(weight), aggr,
                                      num_bags, bag, D, V))
    return out


def embedding_backward(indices, out_grad, weight_grad, aggr=AGGR_NONE, deterministic=False,
                       workspace=True):
    """workspace=True allocates the sort scratch (sorted scatter-add);
    workspace=False passes none (plain atomics, what a caller without scratch gets)."""
    torch = _torch()
    V, D = weight_grad.shape
    if aggr == AGGR_NONE:
        num_bags, bag = indices.numel(), 1
    else:
        bag = indices.shape[-1]
        num_bags = indices.numel() // bag
    ws = None
    ws_bytes = 0
    if workspace or deterministic:
        ws_bytes = lib().ffk_embedding_backward_workspace_bytes(num_bags * bag, V)
        if ws_bytes:
            ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=weight_grad.device)
    check(lib().ffk_embedding_backward(current_stream(), dtype_of(indices), dtype_of(out_grad),
                                       ptr(indices), ptr(out_grad), ptr(weight_grad), aggr,
                                       num_bags, bag, D, V, int(deterministic), ptr(ws),
                                       ws_bytes))
    return weight_grad


def embedding_backward_typed(indices, out_grad, weight_grad, aggr=AGGR_NONE):
    """HALF / DOUBLE (or FLOAT) tables: weight_grad has out_grad's dtype and is added to in that type."""
    V, D = weight_grad.shape
    assert out_grad.dtype == weight_grad.dtype
    if aggr == AGGR_NONE:
        num_bags, bag = indices.numel(), 1
    else:
        bag = indices.shape[-1]
        num_bags = indices.numel() // bag
    check(lib().ffk_embedding_backward_typed(current_stream(), dtype_of(indices), dtype_of(out_grad), ptr(indices),
                                             ptr(out_grad), ptr(weight_grad), aggr, num_bags, bag, D, V))
    return weight_grad


def attention_desc_bshd(q, k, scale, causal, v=None):
    """Descriptor for dense q [B, Sq, H, D], k [B, Skv, H, D], v [B, Skv, H, Dv] tensors."""
    B, Sq, H, D = q.shape
    Skv = k.shape[1]
    Dv = D if v is None else v.shape[3]
    return AttentionDesc(B, H, Sq, Skv, D, Sq * H * D, H * D, Skv * H * D, H * D,
                         Skv * H * Dv, H * Dv, Sq * H * Dv, H * Dv, scale, int(causal), Dv)


def attention_forward(q, k, v, scale, causal, desc=None):
    torch = _torch()
    desc = desc or attention_desc_bshd(q, k, scale, causal, v)
    o = torch.empty(tuple(q.shape[:3]) + (v.shape[3],), dtype=q.dtype, device=q.device)
    lse = torch.empty((desc.batch, desc.heads, desc.seq_q), dtype=torch.float32, device=q.device)
    check(lib().ffk_attention_forward(current_stream(), dtype_of(q), ctypes.byref(desc), ptr(q),
                                      ptr(k), ptr(v), ptr(o), ptr(lse)))
    return o, lse


def attention_backward(q, k, v, o, d_o, lse, scale, causal, desc=None):
    torch = _torch()
    desc = desc or attention_desc_bshd(q, k, scale, causal, v)
    dq = torch.empty_like(q)
    dk = torch.empty_like(k)
    dv = torch.empty_like(v)
    delta = torch.empty_like(lse)
    check(lib().ffk_attention_backward(current_stream(), dtype_of(q), ctypes.byref(desc), ptr(q),
                                       ptr(k), ptr(v), ptr(o), ptr(d_o), ptr(lse), ptr(delta),
                                       ptr(dq), ptr(dk), ptr(dv)))
    return dq, dk, dv


def mha_desc(num_samples, num_heads, q_size, k_size, v_size, q_proj, k_proj, v_proj, o_proj,
             sq, skv, scale=1.0, causal=False):
    return MHADesc(num_samples, num_heads, q_size, k_size, v_size, q_proj, k_proj, v_proj, o_proj,
                   sq, skv, scale, int(causal))


# bits of ffk_mha_backward's `accumulate`
MHA_ACC_INPUT_GRADS, MHA_OVERWRITE_WEIGHT_GRAD = 1, 2


def mha_reserve(desc, dtype, device="cuda"):
    torch = _torch()
    n = lib().ffk_mha_reserve_bytes(ctypes.byref(desc), dtype)
    return torch.empty((n,), dtype=torch.uint8, device=device)


def mha_forward(desc, query, key, value, weight, reserve, out=None):
    torch = _torch()
    if out is None:
        out = torch.empty((desc.num_samples, desc.qo_seq_length, desc.o_proj_size),
                          dtype=query.dtype, device=query.device)
    check(lib().ffk_mha_forward(current_stream(), dtype_of(query), ctypes.byref(desc), ptr(query),
                                ptr(key), ptr(value), ptr(weight), ptr(out), ptr(reserve),
                                reserve.numel()))
    return out


def mha_backward(desc, query, dquery, key, dkey, value, dvalue, weight, dweight, out_grad,
                 reserve, accumulate=False):
    check(lib().ffk_mha_backward(current_stream(), dtype_of(query), ctypes.byref(desc),
                                 ptr(query), ptr(dquery), ptr(key), ptr(dkey), ptr(value),
                                 ptr(dvalue), ptr(weight), ptr(dweight), ptr(out_grad),
                                 ptr(reserve), reserve.numel(), int(accumulate)))
    return dquery, dkey, dvalue, dweight


PARAM_NAMES = ("ln1_gamma", "ln1_beta", "attn_weight", "ln2_gamma", "ln2_beta", "w1", "b1", "w2", "b2")


def encoder_layer_param_shapes(desc):
    """name -> shape of every weight tensor of one encoder layer."""
    E, F, H = desc.d_model, desc.d_ff, desc.heads
    hd = E // H
    return {
        "ln1_gamma": (E,), "ln1_beta": (E,), "attn_weight": (H * hd * 3 * E + E * H * hd,),
        "ln2_gamma": (E,), "ln2_beta": (E,), "w1": (F, E), "b1": (F,), "w2": (E, F), "b2": (E,),
    }


def encoder_layer_params(tensors):
    return EncoderLayerParams(*[ptr(tensors[n]) for n in PARAM_NAMES])


def encoder_layer_workspace(desc, dtype, device="cuda"):
    torch = _torch()
    n = lib().ffk_encoder_layer_workspace_bytes(ctypes.byref(desc), dtype)
    return torch.empty((n,), dtype=torch.uint8, device=device)


def encoder_layer_forward(desc, weights, x, y, workspace):
    check(lib().ffk_encoder_layer_forward(current_stream(), dtype_of(x), ctypes.byref(desc),
                                          ctypes.byref(weights), ptr(x), ptr(y), ptr(workspace),
                                          workspace.numel()))
    return y


def encoder_layer_backward(desc, weights, grads, x, dy, dx, workspace):
    check(lib().ffk_encoder_layer_backward(current_stream(), dtype_of(x), ctypes.byref(desc),
                                           ctypes.byref(weights), ctypes.byref(grads), ptr(x),
                                           ptr(dy), ptr(dx), ptr(workspace), workspace.numel()))
    return dx


def _concat_args(tensors, axis):
    import ctypes
    shape0 = tuple(tensors[0].shape)
    axis = axis if axis >= 0 else len(shape0) + axis
    num_blocks = 1
    for d in shape0[:axis]:
        num_blocks *= d
    blk = []
    for t in tensors:
        sh = tuple(t.shape)
        if len(sh) != len(shape0) or sh[:axis] != shape0[:axis] or sh[axis + 1:] != shape0[axis + 1:]:
            raise ValueError("concat: shapes differ outside the axis")
        n = 1
        for d in sh[axis:]:
            n *= d
        blk.append(n)
    ptrs = (ctypes.c_void_p * len(tensors))(*[ptr(t) for t in tensors])
    blks = (ctypes.c_int64 * len(tensors))(*blk)
    return axis, num_blocks, ptrs, blks


def concat_forward(inputs, axis, out=None):
    """out = concatenation of `inputs` (contiguous tensors of one dtype) along `axis`."""
    torch = _torch()
    axis, num_blocks, ptrs, blks = _concat_args(inputs, axis)
    if out is None:
        shape = list(inputs[0].shape)
        shape[axis] = sum(t.shape[axis] for t in inputs)
        out = torch.empty(shape, dtype=inputs[0].dtype, device=inputs[0].device)
    check(lib().ffk_concat_forward(current_stream(), dtype_of(out), ptr(out), ptrs, blks, len(inputs),
                                   num_blocks))
    return out


def concat_backward(out_grad, input_grads, axis, accumulate=True):
    """input_grads[i] (+)= the slice of out_grad that input i produced."""
    axis, num_blocks, ptrs, blks = _concat_args(input_grads, axis)
    check(lib().ffk_concat_backward(current_stream(), dtype_of(out_grad), ptr(out_grad), ptrs, blks,
                                    len(input_grads), num_blocks, int(accumulate)))
    return input_grads


def transpose_forward(x, perm, out=None):
    """out = x.permute(perm), materialised (x contiguous)."""
    import ctypes
    torch = _torch()
    dims = (ctypes.c_int64 * x.dim())(*x.shape)
    pm = (ctypes.c_int * x.dim())(*perm)
    if out is None:
        out = torch.empty([x.shape[p] for p in perm], dtype=x.dtype, device=x.device)
    check(lib().ffk_transpose_forward(current_stream(), dtype_of(x), ptr(x), ptr(out), x.dim(), dims, pm))
    return out


def transpose_backward(out_grad, in_grad, perm, accumulate=True):
    """in_grad (+)= out_grad moved back through the inverse of `perm`; in_grad has the input's shape."""
    import ctypes
    dims = (ctypes.c_int64 * in_grad.dim())(*in_grad.shape)
    pm = (ctypes.c_int * in_grad.dim())(*perm)
    check(lib().ffk_transpose_backward(current_stream(), dtype_of(out_grad), ptr(out_grad), ptr(in_grad),
                                       in_grad.dim(), dims, pm, int(accumulate)))
    return in_grad


def _gather_view(shape, out_shape, dim):
    dim = dim if dim >= 0 else len(shape) + dim
    outer = 1
    for d in shape[:dim]:
        outer *= d
    stride = 1
    for d in shape[dim + 1:]:
        stride *= d
    return outer, shape[dim], out_shape[dim], stride


def gather_forward(x, index, dim, out=None):
    """torch.gather(x, dim, index) for index of x's shape except along `dim`."""
    torch = _torch()
    outer, ind, outd, stride = _gather_view(tuple(x.shape), tuple(index.shape), dim)
    if out is None:
        out = torch.empty(index.shape, dtype=x.dtype, device=x.device)
    check(lib().ffk_gather_forward(current_stream(), dtype_of(x), dtype_of(index), ptr(x), ptr(index), ptr(out),
                                   outer, ind, outd, stride))
    return out


def gather_backward(out_grad, index, in_grad, dim):
    """in_grad[.., index, ..] += out_grad (fp32, atomics)."""
    outer, ind, outd, stride = _gather_view(tuple(in_grad.shape), tuple(index.shape), dim)
    check(lib().ffk_gather_backward(current_stream(), dtype_of(index), ptr(out_grad), ptr(index), ptr(in_grad),
                                    outer, ind, outd, stride))
    return in_grad


def split_forward(x, sizes, axis):
    """The pieces of x along `axis` with extents `sizes`, as new contiguous tensors."""
    torch = _torch()
    axis = axis if axis >= 0 else x.dim() + axis
    outs = []
    for n in sizes:
        shape = list(x.shape)
        shape[axis] = n
        outs.append(torch.empty(shape, dtype=x.dtype, device=x.device))
    _, num_blocks, ptrs, blks = _concat_args(outs, axis)
    check(lib().ffk_split_forward(current_stream(), dtype_of(x), ptrs, ptr(x), blks, len(outs), num_blocks))
    return outs


def split_backward(out_grads, in_grad, axis, accumulate=True):
    """in_grad (+)= the output gradients side by side along `axis`."""
    axis, num_blocks, ptrs, blks = _concat_args(out_grads, axis)
    check(lib().ffk_split_backward(current_stream(), dtype_of(in_grad), ptr(in_grad), ptrs, blks,
                                   len(out_grads), num_blocks, int(accumulate)))
    return in_grad
