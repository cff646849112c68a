"""The encoder layer composed from oracle operators, rounding to bf16 where the
device stores bf16 (after every operator)."""
import numpy as np


def _r(oracle, a, bf16):
    return oracle.round_bf16(a) if bf16 else np.asarray(a, dtype=np.float32)


def layer_forward_backward(oracle, cfg, params, x, dy, bf16=True):
    """cfg: dict(batch, seq, d_model, heads, d_ff, p, seed, eps, scale, causal,
    pre_ln, gelu).  Returns (y, dx, grads dict)."""
    B, S, E, H, F = cfg["batch"], cfg["seq"], cfg["d_model"], cfg["heads"], cfg["d_ff"]
    T, hd = B * S, E // H
    p, seed, eps = cfg["p"], cfg["seed"], cfg["eps"]
    r = lambda a: _r(oracle, a, bf16)
    GELU, ADD = 67, 28
    desc = oracle.mha_desc(B, H, E, E, E, hd, hd, hd, E, S, S, cfg["scale"], cfg["causal"])
    x2 = x.reshape(T, E)
    dy2 = dy.reshape(T, E)
    g = {}

    def ffn_fwd(inp):
        if cfg["gelu"]:
            f1 = r(oracle.linear_forward(inp, params["w1"], params["b1"]))
            act = r(oracle.element_unary_forward(GELU, f1))
        else:
            f1 = None
            act = r(oracle.linear_forward(inp, params["w1"], params["b1"], activation=0))
        actd = r(oracle.dropout_forward(act, p, seed + 1))
        f2 = r(oracle.linear_forward(actd, params["w2"], params["b2"]))
        f2d = r(oracle.dropout_forward(f2, p, seed + 2))
        return f1, act, actd, f2, f2d

    def ffn_bwd(g_out, inp, f1, act, actd, f2):
        g_f2 = r(oracle.dropout_backward(g_out, p, seed + 2))
        g_actd, dw2, db2 = oracle.linear_backward(f2, g_f2, actd, params["w2"])
        g_actd = r(g_actd)
        g_act = r(oracle.dropout_backward(g_actd, p, seed + 1))
        if cfg["gelu"]:
            g_f1 = r(oracle.element_unary_backward(GELU, act, g_act, f1, accumulate=0))
            g_in, dw1, db1 = oracle.linear_backward(f1, g_f1, inp, params["w1"])
        else:
            g_in, dw1, db1 = oracle.linear_backward(act, g_act, inp, params["w1"], activation=0)
        g.update(w1=r(dw1), b1=r(db1), w2=r(dw2), b2=r(db2))
        return r(g_in)

    if cfg["pre_ln"]:
        h1, m1, s1 = oracle.layer_norm_forward(x2, params["ln1_gamma"], params["ln1_beta"], eps)
        h1 = r(h1)
        attn = oracle.mha_forward(desc, h1.reshape(B, S, E), h1.reshape(B, S, E), h1.reshape(B, S, E),
                                  params["attn_weight"], bf16_mode=bf16).reshape(T, E)
        attnd = r(oracle.dropout_forward(attn, p, seed + 0))
        x1 = r(oracle.element_binary_forward(ADD, attnd, x2))
        h2, m2, s2 = oracle.layer_norm_forward(x1, params["ln2_gamma"], params["ln2_beta"], eps)
        h2 = r(h2)
        f1, act, actd, f2, f2d = ffn_fwd(h2)
        y = r(oracle.element_binary_forward(ADD, x1, f2d))
        # backward
        g_h2 = ffn_bwd(dy2, h2, f1, act, actd, f2)
        g_x1, dg2, db2 = oracle.layer_norm_backward(g_h2, x1, m2, s2, params["ln2_gamma"])
        g_x1 = r(r(g_x1) + dy2)
        g_attn = r(oracle.dropout_backward(g_x1, p, seed + 0))
        h1b = h1.reshape(B, S, E)
        dq, dk, dv, dw = oracle.mha_backward(desc, h1b, h1b, h1b, params["attn_weight"],
                                             g_attn.reshape(B, S, E), bf16_mode=bf16)
        g_h1 = r((dq + dk + dv).reshape(T, E))
        dx, dg1, db1 = oracle.layer_norm_backward(g_h1, x2, m1, s1, params["ln1_gamma"])
        dx = r(r(dx) + g_x1)
    else:
        xb = x2.reshape(B, S, E)
        attn = oracle.mha_forward(desc, xb, xb, xb, params["attn_weight"], bf16_mode=bf16).reshape(T, E)
        h1 = r(oracle.element_binary_forward(ADD, attn, x2))
        x1, m1, s1 = oracle.layer_norm_forward(h1, params["ln1_gamma"], params["ln1_beta"], eps)
        x1 = r(x1)
        f1, act, actd, f2, f2d = ffn_fwd(x1)
        pre2 = r(oracle.element_binary_forward(ADD, x1, f2d))
        y, m2, s2 = oracle.layer_norm_forward(pre2, params["ln2_gamma"], params["ln2_beta"], eps)
        y = r(y)
        g_sum, dg2, db2 = oracle.layer_norm_backward(dy2, pre2, m2, s2, params["ln2_gamma"])
        g_sum = r(g_sum)
        g_in = ffn_bwd(g_sum, x1, f1, act, actd, f2)
        g_x1 = r(g_in + g_sum)
        g_h1, dg1, db1 = oracle.layer_norm_backward(g_x1, h1, m1, s1, params["ln1_gamma"])
        g_h1 = r(g_h1)
        dq, dk, dv, dw = oracle.mha_backward(desc, xb, xb, xb, params["attn_weight"],
                                             g_h1.reshape(B, S, E), bf16_mode=bf16)
        dx = r(r((dq + dk + dv).reshape(T, E)) + g_h1)
    g.update(ln1_gamma=r(dg1), ln1_beta=r(db1), ln2_gamma=r(dg2), ln2_beta=r(db2), attn_weight=r(dw))
    return y.reshape(x.shape), dx.reshape(x.shape), g


def make_params(rng, cfg, bf16_round):
    E, F, H = cfg["d_model"], cfg["d_ff"], cfg["heads"]
    hd = E // H
    n = lambda *s: bf16_round((rng.standard_normal(s) * 0.02).astype(np.float32))
    return {
        "ln1_gamma": bf16_round(1 + 0.02 * rng.standard_normal(E)), "ln1_beta": n(E),
        "attn_weight": n(H * hd * 3 * E + E * H * hd),
        "ln2_gamma": bf16_round(1 + 0.02 * rng.standard_normal(E)), "ln2_beta": n(E),
        "w1": n(F, E), "b1": n(F), "w2": n(E, F), "b2": n(E),
    }
