"""ctypes binding of the CPU oracle (oracle/libffk_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of bench.py.  The product package never imports this module.
Arrays are numpy float32 (C-contiguous) unless stated.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libffk_oracle.so")
_lib = None

c_i64 = ctypes.c_int64
c_f = ctypes.c_float
c_int = ctypes.c_int
c_u64 = ctypes.c_uint64
c_p = ctypes.c_void_p


def build():
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return _LIB_PATH


class MHADesc(ctypes.Structure):
    _fields_ = [
        ("num_samples", c_i64), ("num_heads", c_i64),
        ("q_size", c_i64), ("k_size", c_i64), ("v_size", c_i64),
        ("q_proj_size", c_i64), ("k_proj_size", c_i64), ("v_proj_size", c_i64),
        ("o_proj_size", c_i64),
        ("qo_seq_length", c_i64), ("kv_seq_length", c_i64),
        ("scale", c_f), ("causal", c_int),
    ]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_round_bf16.restype = c_f
        _lib.orc_round_bf16.argtypes = [c_f]
        _lib.orc_offset.restype = c_i64
    return _lib


def set_num_threads(n):
    """Threads for the oracle's row- and head-parallel loops (same bits for any count)."""
    lib().orc_set_num_threads(c_int(int(n)))


def max_threads():
    return int(lib().orc_get_max_threads())


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _p(a):
    return None if a is None else a.ctypes.data_as(c_p)


def round_bf16(a):
    a = _f32(a).copy()
    lib().orc_round_bf16_array(_p(a), c_i64(a.size))
    return a


def offset(dims, coord):
    d = np.asarray(dims, dtype=np.int64)
    c = np.asarray(coord, dtype=np.int64)
    return int(lib().orc_offset(_p(d), c_int(len(d)), _p(c)))


def matmul(lhs, rhs):
    lhs, rhs = _f32(lhs), _f32(rhs)
    M, K = lhs.shape
    K2, N = rhs.shape
    assert K == K2
    out = np.empty((M, N), np.float32)
    lib().orc_matmul(_p(lhs), _p(rhs), _p(out), c_i64(M), c_i64(K), c_i64(N))
    return out


def transpose(a):
    a = _f32(a)
    out = np.empty((a.shape[1], a.shape[0]), np.float32)
    lib().orc_transpose(_p(a), _p(out), c_i64(a.shape[0]), c_i64(a.shape[1]))
    return out


def broadcast(a, out_dims):
    a = _f32(a)
    ind = np.asarray(a.shape, dtype=np.int64)
    outd = np.asarray(out_dims, dtype=np.int64)
    out = np.empty(tuple(out_dims), np.float32)
    lib().orc_broadcast(_p(a), _p(ind), c_int(a.ndim), _p(out), _p(outd), c_int(len(outd)))
    return out


def reduce_dim(a, dim):
    a = _f32(a)
    d = np.asarray(a.shape, dtype=np.int64)
    out_shape = a.shape[:dim] + a.shape[dim + 1:]
    out = np.empty(out_shape, np.float32)
    lib().orc_reduce_dim(_p(a), _p(d), c_int(a.ndim), c_int(dim), _p(out))
    return out


def relu(a):
    a = _f32(a)
    out = np.empty_like(a)
    lib().orc_relu(_p(a), _p(out), c_i64(a.size))
    return out


def scale(a, c):
    a = _f32(a)
    out = np.empty_like(a)
    lib().orc_scale(_p(a), c_f(c), _p(out), c_i64(a.size))
    return out


def linear_forward(x, w, b=None, activation=-1):
    x, w = _f32(x), _f32(w)
    b = None if b is None else _f32(b)
    batch, in_dim = x.shape
    out_dim = w.shape[0]
    y = np.empty((batch, out_dim), np.float32)
    rc = lib().orc_linear_forward(c_int(activation), _p(x), _p(y), _p(w), _p(b),
                                  c_i64(batch), c_i64(in_dim), c_i64(out_dim))
    if rc:
        raise ValueError("Unhandled activation function")
    return y


def linear_backward(y, dy, x, w, activation=-1, relu_grad_mode=0, use_bias=True):
    y, dy, x, w = _f32(y), _f32(dy), _f32(x), _f32(w)
    batch, in_dim = x.shape
    out_dim = w.shape[0]
    dx = np.empty_like(x)
    dw = np.empty_like(w)
    db = np.empty((out_dim,), np.float32) if use_bias else None
    rc = lib().orc_linear_backward(c_int(activation), c_int(relu_grad_mode), _p(y), _p(dy),
                                   _p(x), _p(dx), _p(w), _p(dw), _p(db),
                                   c_i64(batch), c_i64(in_dim), c_i64(out_dim))
    if rc:
        raise ValueError("Unhandled activation function")
    return dx, dw, db


def linear_l2_regularizer_grad(w, dw, lam):
    """Returns dw + lam * w (the reference adds the term once per backward call)."""
    w = _f32(w)
    out = np.array(_f32(dw), copy=True)
    lib().orc_linear_l2_regularizer_grad(_p(w), _p(out), c_i64(w.size), c_f(lam))
    return out


def gemm_f64(A, B, trans_a=False, trans_b=False):
    A, B = _f32(A), _f32(B)
    M = A.shape[1] if trans_a else A.shape[0]
    K = A.shape[0] if trans_a else A.shape[1]
    N = B.shape[0] if trans_b else B.shape[1]
    C = np.empty((M, N), np.float32)
    lib().orc_gemm_f64(c_int(int(trans_a)), c_int(int(trans_b)), c_i64(M), c_i64(N), c_i64(K),
                       _p(A), _p(B), _p(C))
    return C


def element_unary_forward(op, x, scalar=0.0):
    x = _f32(x)
    y = np.empty_like(x)
    rc = lib().orc_element_unary_forward(c_int(op), c_f(scalar), _p(x), _p(y), c_i64(x.size))
    if rc:
        raise ValueError("unhandled unary op %d" % op)
    return y


def element_unary_backward(op, y, dy, x, dx_init=None, scalar=0.0, accumulate=-1):
    y, dy, x = _f32(y), _f32(dy), _f32(x)
    dx = np.zeros_like(x) if dx_init is None else _f32(dx_init).copy()
    rc = lib().orc_element_unary_backward(c_int(op), c_f(scalar), _p(y), _p(dy), _p(x), _p(dx),
                                          c_i64(x.size), c_int(accumulate))
    if rc:
        raise ValueError("unhandled unary op %d" % op)
    return dx


def element_binary_forward(op, l, r, out_shape=None):
    l, r = _f32(l), _f32(r)
    shape = out_shape if out_shape is not None else (l.shape if l.size >= r.size else r.shape)
    out = np.empty(shape, np.float32)
    rc = lib().orc_element_binary_forward(c_int(op), _p(l), _p(r), _p(out), c_i64(out.size),
                                          c_i64(l.size), c_i64(r.size))
    if rc:
        raise ValueError("unhandled binary op %d" % op)
    return out


def element_binary_backward(op, g, l, r, dl_init=None, dr_init=None, accumulate=0):
    g, l, r = _f32(g), _f32(l), _f32(r)
    dl = np.zeros_like(g) if dl_init is None else _f32(dl_init).copy()
    dr = np.zeros_like(g) if dr_init is None else _f32(dr_init).copy()
    rc = lib().orc_element_binary_backward(c_int(op), _p(g), _p(l), _p(r), _p(dl), _p(dr),
                                           c_i64(g.size), c_int(accumulate))
    if rc:
        raise ValueError("unhandled binary op %d" % op)
    return dl, dr


def element_binary_backward_broadcast(op, g, l, r, dl_init=None, dr_init=None, accumulate=0):
    """Gradients when an operand was broadcast over the leading dims (operand index = output index
    modulo the operand's size): what lib/kernels/src/cuda/ops/element_binary_kernels.cu:268-396 asks
    cuDNN for -- add / sub: reduce dy (sub negates the rhs); mul: reduce dy * other operand -- each
    added into (accumulate) or stored to the operand's gradient.  Sums in float64, rounded once."""
    g, l, r = _f32(g), _f32(l), _f32(r)
    n = g.size
    OP_EW_ADD, OP_EW_MUL, OP_EW_SUB = 28, 29, 35  # OperatorType ordinals (op-attrs/operator_type.dtg.toml order)

    def spread(a):
        return np.resize(a.reshape(-1), n).astype(np.float64)  # a[i % a.size]

    gl = g.reshape(-1).astype(np.float64)
    if op == OP_EW_ADD:
        tl, tr = gl, gl
    elif op == OP_EW_SUB:
        tl, tr = gl, -gl
    elif op == OP_EW_MUL:
        tl, tr = gl * spread(r), gl * spread(l)
    else:
        raise ValueError("no broadcast gradient for binary op %d" % op)
    out = []
    for term, operand, init in ((tl, l, dl_init), (tr, r, dr_init)):
        red = term.reshape(-1, operand.size).sum(axis=0)
        if accumulate and init is not None:
            red = red + _f32(init).reshape(-1).astype(np.float64)
        out.append(red.astype(np.float32).reshape(operand.shape))
    return out[0], out[1]


def layer_norm_forward(x, gamma, beta, eps):
    x = _f32(x)
    M, N = x.shape
    gamma = None if gamma is None else _f32(gamma)
    beta = None if beta is None else _f32(beta)
    y = np.empty_like(x)
    mean = np.empty((M,), np.float32)
    rstd = np.empty((M,), np.float32)
    lib().orc_layer_norm_forward(_p(x), _p(y), _p(gamma), _p(beta), _p(mean), _p(rstd),
                                 c_i64(M), c_i64(N), c_f(eps))
    return y, mean, rstd


def layer_norm_backward(dy, x, mean, rstd, gamma, dx_init=None):
    dy, x, mean, rstd = _f32(dy), _f32(x), _f32(mean), _f32(rstd)
    M, N = x.shape
    gamma = None if gamma is None else _f32(gamma)
    dx = np.zeros_like(x) if dx_init is None else _f32(dx_init).copy()
    dg = np.empty((N,), np.float32)
    db = np.empty((N,), np.float32)
    lib().orc_layer_norm_backward(_p(dy), _p(x), _p(mean), _p(rstd), _p(gamma), _p(dx), _p(dg),
                                  _p(db), c_i64(M), c_i64(N), c_int(0 if dx_init is None else 1))
    return dx, dg, db


def softmax_forward(x, outer, dim, inner):
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_softmax_forward(_p(x), _p(y), c_i64(outer), c_i64(dim), c_i64(inner))
    return y


def softmax_backward(y, dy, outer, dim, inner):
    y, dy = _f32(y), _f32(dy)
    dx = np.empty_like(y)
    lib().orc_softmax_backward(_p(y), _p(dy), _p(dx), c_i64(outer), c_i64(dim), c_i64(inner))
    return dx


def philox4x32_10(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32)
    k = np.asarray(key, dtype=np.uint32)
    out = np.empty((4,), np.uint32)
    lib().orc_philox4x32_10(_p(c), _p(k), _p(out))
    return out


def dropout_mask(n, rate, seed, offset=0):
    m = np.empty((n,), np.uint8)
    lib().orc_dropout_mask(_p(m), c_i64(n), c_f(rate), c_u64(seed), c_u64(offset))
    return m


def dropout_forward(x, rate, seed, offset=0):
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_dropout_forward(_p(x), _p(y), c_i64(x.size), c_f(rate), c_u64(seed), c_u64(offset))
    return y


def dropout_backward(dy, rate, seed, offset=0, dx_init=None):
    dy = _f32(dy)
    dx = np.zeros_like(dy) if dx_init is None else _f32(dx_init).copy()
    lib().orc_dropout_backward(_p(dy), _p(dx), c_i64(dy.size), c_f(rate), c_u64(seed),
                               c_u64(offset), c_int(0 if dx_init is None else 1))
    return dx


def embedding_forward(indices, weight, aggr=-1):
    idx = np.ascontiguousarray(indices, dtype=np.int64)
    weight = _f32(weight)
    if idx.ndim == 1:
        idx2 = idx.reshape(-1, 1)
    else:
        idx2 = idx.reshape(-1, idx.shape[-1]) if aggr >= 0 else idx.reshape(-1, 1)
    num_bags, bag = idx2.shape
    V, D = weight.shape
    out = np.empty((num_bags, D), np.float32)
    rc = lib().orc_embedding_forward(_p(idx2), _p(out), _p(weight), c_int(aggr), c_i64(num_bags),
                                     c_i64(bag), c_i64(D), c_i64(V))
    if rc:
        raise ValueError("embedding_forward failed rc=%d" % rc)
    return out


def embedding_backward(indices, out_grad, num_entries, aggr=-1, f64=False, dw_init=None):
    idx = np.ascontiguousarray(indices, dtype=np.int64)
    g = _f32(out_grad)
    if idx.ndim == 1 or aggr < 0:
        idx2 = idx.reshape(-1, 1)
    else:
        idx2 = idx.reshape(-1, idx.shape[-1])
    num_bags, bag = idx2.shape
    D = g.shape[-1]
    dw = np.zeros((num_entries, D), np.float32) if dw_init is None else _f32(dw_init).copy()
    fn = lib().orc_embedding_backward_f64 if f64 else lib().orc_embedding_backward
    rc = fn(_p(idx2), _p(g), _p(dw), c_int(aggr), c_i64(num_bags), c_i64(bag), c_i64(D),
            c_i64(num_entries))
    if rc:
        raise ValueError("embedding_backward failed rc=%d" % rc)
    return dw


def _bags(indices, aggr):
    idx = np.ascontiguousarray(indices, dtype=np.int64)
    if idx.ndim == 1 or aggr < 0:
        return idx.reshape(-1, 1)
    return idx.reshape(-1, idx.shape[-1])


def embedding_forward_typed(indices, weight, aggr=-1):
    """The reference's HALF / DOUBLE instantiations (embedding_kernels.cu:48-125 with TD = half or
    double): the bag is summed entry by entry in the table's own type (numpy's float16 add is the
    correctly rounded one: two halves add exactly in the float32 it goes through unless one is
    below an eighth of the other's last place, where no rounding boundary is near); AVG
    multiplies the sum by TD(1.0f / bag) -- once, the same true average as orc_embedding_forward,
    not the reference's multiplication inside the loop."""
    weight = np.asarray(weight)
    assert weight.dtype in (np.float16, np.float64)
    idx2 = _bags(indices, aggr)
    num_bags, bag = idx2.shape
    if idx2.min() < 0 or idx2.max() >= weight.shape[0]:
        raise ValueError("embedding_forward_typed: index out of range")
    acc = np.zeros((num_bags, weight.shape[1]), weight.dtype)
    for j in range(bag):
        acc = (acc + weight[idx2[:, j]]).astype(weight.dtype)
    if aggr == 1:
        acc = (acc * weight.dtype.type(np.float32(1.0) / np.float32(bag))).astype(weight.dtype)
    return acc


def embedding_backward_typed(indices, out_grad, num_entries, aggr=-1, dw_init=None):
    """embedding_kernels.cu:128-317 with TD = half or double and the atomics replaced by adds in
    lookup order: weight_grad[row] += out_grad[bag] (* TD(1.0f / bag) for AVG), every add rounded
    to TD.  (The device's order is not fixed: tests use sums that are exact in TD.)"""
    g = np.asarray(out_grad)
    assert g.dtype in (np.float16, np.float64)
    idx2 = _bags(indices, aggr)
    num_bags, bag = idx2.shape
    dw = np.zeros((num_entries, g.shape[-1]), g.dtype) if dw_init is None else np.array(dw_init, dtype=g.dtype)
    if aggr == 1:
        g = (g * g.dtype.type(np.float32(1.0) / np.float32(bag))).astype(g.dtype)
    for b in range(num_bags):
        for j in range(bag):
            row = idx2[b, j]
            if row < 0 or row >= num_entries:
                raise ValueError("embedding_backward_typed: index out of range")
            dw[row] = (dw[row] + g[b]).astype(g.dtype)
    return dw


def attention_forward(q, k, v, scale, causal, bf16_mode=False):
    """q [B,Sq,H,D], k [B,Skv,H,D], v [B,Skv,H,Dv] -> o [B,Sq,H,Dv], lse [B,H,Sq]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, Sq, H, D = q.shape
    Skv, Dv = k.shape[1], v.shape[3]
    o = np.empty((B, Sq, H, Dv), np.float32)
    lse = np.empty((B, H, Sq), np.float32)
    lib().orc_attention_forward(_p(q), _p(k), _p(v), _p(o), _p(lse), c_i64(B), c_i64(H),
                                c_i64(Sq), c_i64(Skv), c_i64(D), c_i64(Dv), c_f(scale),
                                c_int(int(causal)), c_int(int(bf16_mode)))
    return o, lse


def attention_backward(q, k, v, d_o, scale, causal):
    q, k, v, d_o = _f32(q), _f32(k), _f32(v), _f32(d_o)
    B, Sq, H, D = q.shape
    Skv, Dv = k.shape[1], v.shape[3]
    dq = np.empty_like(q)
    dk = np.empty_like(k)
    dv = np.empty_like(v)
    lib().orc_attention_backward(_p(q), _p(k), _p(v), _p(d_o), _p(dq), _p(dk), _p(dv), c_i64(B),
                                 c_i64(H), c_i64(Sq), c_i64(Skv), c_i64(D), c_i64(Dv), c_f(scale),
                                 c_int(int(causal)))
    return dq, dk, dv


def mha_desc(num_samples, num_heads, q_size, k_size, v_size, q_proj, k_proj, v_proj, o_proj,
             sq, skv, scale=1.0, causal=False):
    return MHADesc(num_samples, num_heads, q_size, k_size, v_size, q_proj, k_proj, v_proj, o_proj,
                   sq, skv, scale, int(causal))


def mha_forward(desc, query, key, value, weight, bf16_mode=False):
    query, key, value, weight = _f32(query), _f32(key), _f32(value), _f32(weight)
    out = np.empty((desc.num_samples, desc.qo_seq_length, desc.o_proj_size), np.float32)
    lib().orc_mha_forward(ctypes.byref(desc), _p(query), _p(key), _p(value), _p(weight), _p(out),
                          c_int(int(bf16_mode)))
    return out


def mha_backward(desc, query, key, value, weight, out_grad, bf16_mode=False):
    query, key, value, weight, out_grad = map(_f32, (query, key, value, weight, out_grad))
    dq = np.empty_like(query)
    dk = np.empty_like(key)
    dv = np.empty_like(value)
    dw = np.zeros_like(weight)
    lib().orc_mha_backward(ctypes.byref(desc), _p(query), _p(key), _p(value), _p(weight),
                           _p(out_grad), _p(dq), _p(dk), _p(dv), _p(dw), c_int(int(bf16_mode)))
    return dq, dk, dv, dw


def sgd_update(w, grad, lr, momentum=0.0, nesterov=False, weight_decay=0.0, v=None, replicas=1):
    """Returns (w_new, v_new); grad holds `replicas` copies of length w.size back to back."""
    w = _f32(w).copy()
    g = _f32(grad)
    vv = None if v is None else _f32(v).copy()
    lib().orc_sgd_update(c_f(lr), c_f(momentum), c_int(int(nesterov)), c_f(weight_decay), _p(g),
                         c_i64(w.size), c_int(replicas), _p(w), _p(vv))
    return w, vv


def adam_update(w, grad, m, v, alpha_t, beta1=0.9, beta2=0.999, weight_decay=0.0, epsilon=1e-8,
                replicas=1):
    """Returns (w_new, m_new, v_new)."""
    w, m, v = _f32(w).copy(), _f32(m).copy(), _f32(v).copy()
    g = _f32(grad)
    lib().orc_adam_update(c_f(alpha_t), c_f(beta1), c_f(beta2), c_f(weight_decay), c_f(epsilon),
                          _p(g), c_i64(w.size), c_int(replicas), _p(w), _p(v), _p(m))
    return w, m, v


def sparse_cce_loss_backward(logit, label, num_samples, num_classes, k, scale_factor):
    logit = _f32(logit)
    label = np.ascontiguousarray(label, dtype=np.int32)
    out = np.empty_like(logit)
    lib().orc_sparse_cce_loss_backward(_p(out), _p(logit), _p(label), c_i64(logit.size),
                                       c_i64(num_samples), c_i64(num_classes), c_int(k),
                                       c_f(scale_factor))
    return out


def difference_loss_backward(logit, label, scale_factor):
    logit, label = _f32(logit), _f32(label)
    out = np.empty_like(logit)
    lib().orc_difference_loss_backward(_p(out), _p(logit), _p(label), c_i64(logit.size),
                                       c_f(scale_factor))
    return out


def identity_loss_backward(shape, scale_factor):
    out = np.empty(shape, np.float32)
    lib().orc_identity_loss_backward(_p(out), c_i64(out.size), c_f(scale_factor))
    return out


def cast(x, out_dtype):
    """static_cast element by element (cast_kernels_cpu.cc:6-11); numpy's astype
    is the same conversion for the type pairs used here."""
    return np.ascontiguousarray(x).astype(out_dtype)


def _concat_blocks(shapes, axis):
    axis = axis if axis >= 0 else len(shapes[0]) + axis
    num_blocks = int(np.prod(shapes[0][:axis], dtype=np.int64))
    blk = [int(np.prod(sh[axis:], dtype=np.int64)) for sh in shapes]
    return axis, num_blocks, blk


def concat_forward(inputs, axis):
    """concat_kernels.cu:36-66: every input is copied into its column window of the
    [num_blocks, sum blk] view of the output."""
    ins = [_f32(a) for a in inputs]
    axis, num_blocks, blk = _concat_blocks([a.shape for a in ins], axis)
    shape = list(ins[0].shape)
    shape[axis] = sum(a.shape[axis] for a in ins)
    out = np.empty(shape, np.float32)
    ptrs = (ctypes.c_void_p * len(ins))(*[a.ctypes.data for a in ins])
    blks = (c_i64 * len(ins))(*blk)
    lib().orc_concat_forward(_p(out), ptrs, blks, ctypes.c_int(len(ins)), c_i64(num_blocks))
    return out


def concat_backward(out_grad, input_grads, axis, accumulate=True):
    """Returns the new input gradients (concat_kernels.cu:68-97 adds into them)."""
    g = _f32(out_grad)
    dins = [_f32(a).copy() for a in input_grads]
    axis, num_blocks, blk = _concat_blocks([a.shape for a in dins], axis)
    ptrs = (ctypes.c_void_p * len(dins))(*[a.ctypes.data for a in dins])
    blks = (c_i64 * len(dins))(*blk)
    lib().orc_concat_backward(_p(g), ptrs, blks, ctypes.c_int(len(dins)), c_i64(num_blocks),
                              ctypes.c_int(1 if accumulate else 0))
    return dins


def transpose_nd(x, perm, into=None):
    """out = x permuted (output dim i = input dim perm[i]); with `into`, added to it."""
    x = _f32(x)
    nd = x.ndim
    out = np.empty([x.shape[p] for p in perm], np.float32) if into is None else _f32(into).copy()
    dims = (c_i64 * nd)(*x.shape)
    pm = (ctypes.c_int * nd)(*perm)
    lib().orc_transpose_nd(_p(x), _p(out), ctypes.c_int(nd), dims, pm, ctypes.c_int(0 if into is None else 1))
    return out


def _gather_view(shape, out_shape, dim):
    dim = dim if dim >= 0 else len(shape) + dim
    outer = int(np.prod(shape[:dim], dtype=np.int64))
    stride = int(np.prod(shape[dim + 1:], dtype=np.int64))
    return outer, int(shape[dim]), int(out_shape[dim]), stride


def gather_forward(x, index, dim):
    x = _f32(x)
    idx = np.ascontiguousarray(index, dtype=np.int64)
    outer, ind, outd, stride = _gather_view(x.shape, idx.shape, dim)
    out = np.empty(idx.shape, np.float32)
    lib().orc_gather_forward(_p(x), idx.ctypes.data_as(ctypes.c_void_p), _p(out), c_i64(outer), c_i64(ind),
                             c_i64(outd), c_i64(stride))
    return out


def gather_backward(out_grad, index, in_grad, dim):
    """Returns in_grad with the gradient scattered into it."""
    g = _f32(out_grad)
    idx = np.ascontiguousarray(index, dtype=np.int64)
    din = _f32(in_grad).copy()
    outer, ind, outd, stride = _gather_view(din.shape, idx.shape, dim)
    lib().orc_gather_backward(_p(g), idx.ctypes.data_as(ctypes.c_void_p), _p(din), c_i64(outer), c_i64(ind),
                              c_i64(outd), c_i64(stride))
    return din
