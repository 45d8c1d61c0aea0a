"""Canonical IR text of each evaluated computation, built from the dimensions
in a tensor-metadata config.

The reference reads its IR from per-case text files produced by an
equality-saturation search that is not part of its repository
(convert_eval_rms.py:25-29); these builders write one representative
expression per family in the same grammar (codegen/IrParser.py), so that the
`convert_*` entry points work out of the box.
"""


def _ld(kind, names, *idx):
    return "(load (%s %s) (index %s))" % (kind, names, " ".join(idx))


def _st(kind, names, value, *idx):
    return "(store (%s %s) %s (index %s))" % (kind, names, value, " ".join(idx))


def _seq(*items):
    items = [i for i in items if i]
    out = items[-1]
    for it in reversed(items[:-1]):
        out = "(seq %s %s)" % (it, out)
    return out


FT, TN, TK, TP, EN = "fulltile", "(tile n)", "(tile k)", "(tile p)", "(elem n)"


def attention_ir(variant, M, N, D, P, prenorm=False, qknorm=False, tau=1.5):
    """QKV projection + cache append + attention for one head per ploop tile."""
    L = P + M
    acc = _ld("tensor", "Q1,K1,V1", FT, TN)
    proj = _st("tensor", "Q1,K1,V1",
               "(+ (x %s 1) (* %s %s))" % (acc, _ld("input", "X", FT, TK), _ld("input", "WQ,WK,WV", TK, TN)), FT, TN)
    if prenorm:
        x2 = _st("tensor", "X2", "(+ (x %s 1) (rsum (sqr %s) 1))" % (_ld("tensor", "X2", FT), _ld("input", "X", FT, TK)), FT)
        k_loop = "(sloop 0 %d tile_k k %s)" % (N, _seq(x2, proj))
        scale = _st("tensor", "Q1,K1,V1",
                    "(/ %s (bcast (sqrt (/ %s %d)) 1))" % (acc, _ld("tensor", "X2", FT), N), FT, TN)
    else:
        k_loop = "(sloop 0 %d tile_k k %s)" % (N, proj)
        scale = None
    heads = _st("tensor", "Q,K,V", "(permute3 (unsqueeze %s 1) 1 0 2)" % acc, EN, FT, FT)
    q_name, k_name = "Q", "K"
    norm = None
    if qknorm:
        qk = _ld("tensor", "Q,K", EN, FT, FT)
        norm = _st("tensor", "Q_norm,K_norm", "(/ %s (bcast (sqrt (/ (rsum (sqr %s) 2) %d)) 2))" % (qk, qk, D), EN, FT, FT)
        q_name, k_name = "Q_norm", "K_norm"
    append = _st("input", "K_cache,V_cache", _ld("tensor", "%s,V" % k_name, EN, FT, FT), EN, "(const_tile %d %d)" % (P, M), FT)
    q = _ld("tensor", q_name, EN, FT, FT)
    kt = "(permute3 %s 0 2 1)" % _ld("input", "K_cache", EN, TP, FT)
    c_exp = _ld("tensor", "C_exp", EN, FT, TP)
    c_sum = _ld("tensor", "C_sum", EN, FT)
    o = _ld("tensor", "O", EN, FT, FT)
    v = _ld("input", "V_cache", EN, TP, FT)
    st_exp = _st("tensor", "C_exp", "(exp (* %s %s))" % (q, kt), EN, FT, TP)
    st_sum = _st("tensor", "C_sum", "(+ (x %s 1) (rsum %s 2))" % (c_sum, c_exp), EN, FT)
    st_o = _st("tensor", "O", "(+ (x %s 1) (* %s %s))" % (o, c_exp, v), EN, FT, FT)
    finish = _st("tensor", "O", "(/ %s (bcast %s 2))" % (o, c_sum), EN, FT, FT)
    out = _st("output", "O2", "(squeeze (permute3 %s 1 0 2) 1)" % o, FT, TN)
    if variant == "vanilla":
        body = [k_loop, scale, heads, norm, append, "(sloop 0 %d tile_p p %s)" % (L, _seq(st_exp, st_sum, st_o)), finish, out]
    elif variant == "roco":
        c_div = _ld("tensor", "C_div", EN, FT, TP)
        pass2 = _seq(_st("tensor", "C_div", "(/ %s (bcast %s 2))" % (c_exp, c_sum), EN, FT, TP),
                     _st("tensor", "O", "(+ (x %s 1) (* %s %s))" % (o, c_div, v), EN, FT, FT),
                     _st("output", "C_out1", "(rsum %s 1)" % c_div, EN, TP),
                     _st("output", "C_out2", "(rsum (sqr %s) 1)" % c_div, EN, TP))
        body = [k_loop, scale, heads, norm, append, "(sloop 0 %d tile_p p %s)" % (L, _seq(st_exp, st_sum)),
                "(sloop 0 %d tile_p p %s)" % (L, pass2), out]
    elif variant == "keyformer":
        c = _ld("tensor", "C", EN, FT, TP)
        pert = _ld("tensor", "C_perturb", EN, FT, TP)
        exp_p = _ld("tensor", "C_exp_perturb", EN, FT, TP)
        sum_p = _ld("tensor", "C_sum_perturb", EN, FT)
        pass1 = _seq(_st("tensor", "C", "(* %s %s)" % (q, kt), EN, FT, TP),
                     _st("tensor", "C_perturb", "(/ (+ %s %s) %s)" % (c, _ld("input", "noise", EN, FT, TP), repr(float(tau))), EN, FT, TP),
                     _st("tensor", "C_exp,C_exp_perturb", "(exp %s)" % _ld("tensor", "C,C_perturb", EN, FT, TP), EN, FT, TP),
                     _st("tensor", "C_sum,C_sum_perturb",
                         "(+ (x %s 1) (rsum %s 2))" % (_ld("tensor", "C_sum,C_sum_perturb", EN, FT),
                                                       _ld("tensor", "C_exp,C_exp_perturb", EN, FT, TP)), EN, FT),
                     st_o)
        pass2 = _st("output", "C_out", "(rsum (/ %s (bcast %s 2)) 1)" % (exp_p, sum_p), EN, TP)
        body = [k_loop, scale, heads, norm, append, "(sloop 0 %d tile_p p %s)" % (L, pass1),
                "(sloop 0 %d tile_p p %s)" % (L, pass2), finish, out]
    else:
        raise ValueError("unknown variant %r" % variant)
    return "(ploop 0 %d %d n %s)" % (N, D, _seq(*body))


def ffn_ir(N, P, falcon_tail=False):
    """Output projection + residual, RMSNorm folded into the gate/up GEMMs,
    SwiGLU, down projection (+ residual + RMSNorm): one kernel per stage."""
    k1 = "(ploop 0 %d tile_n n %s)" % (N, _seq(
        "(sloop 0 %d tile_k k %s)" % (N, _st("tensor", "attn_O1", "(+ (x %s 1) (* %s %s))" % (
            _ld("tensor", "attn_O1", FT, TN), _ld("input", "O2", FT, TK), _ld("input", "WO", TK, TN)), FT, TN)),
        _st("tensor", "attn_O2", "(+ %s %s)" % (_ld("input", "X", FT, TN), _ld("tensor", "attn_O1", FT, TN)), FT, TN)))
    a2k = _ld("tensor", "attn_O2", FT, TK)
    o3 = _ld("tensor", "attn_O3", FT)
    inner = _seq(_st("tensor", "attn_O3", "(+ (x %s 1) (rsum (sqr %s) 1))" % (o3, a2k), FT),
                 _st("tensor", "FF1a,FF1b", "(+ (x %s 1) (* %s %s))" % (
                     _ld("tensor", "FF1a,FF1b", FT, TP), a2k, _ld("input", "WFF1a,WFF1b", TK, TP)), FT, TP))
    ab = _ld("tensor", "FF1a,FF1b", FT, TP)
    k2 = "(ploop 0 %d tile_p p %s)" % (P, _seq(
        "(sloop 0 %d tile_k k %s)" % (N, inner),
        _st("tensor", "FF1a,FF1b", "(/ %s (bcast (sqrt (/ %s %d)) 1))" % (ab, o3, N), FT, TP),
        _st("tensor", "FF1", "(x (x %s (sigmoid %s)) %s)" % (
            _ld("tensor", "FF1b", FT, TP), _ld("tensor", "FF1b", FT, TP), _ld("tensor", "FF1a", FT, TP)), FT, TP)))
    down_target = ("tensor", "FF2") if falcon_tail else ("output", "FF2")
    k3 = "(ploop 0 %d tile_n n (sloop 0 %d tile_p p %s))" % (N, P, _st(
        down_target[0], down_target[1], "(+ (x %s 1) (* %s %s))" % (
            _ld(down_target[0], down_target[1], FT, TN), _ld("tensor", "FF1", FT, TP), _ld("input", "WFF2", TP, TN)), FT, TN))
    if not falcon_tail:
        return _seq(k1, k2, k3)
    a2n = _ld("tensor", "attn_O2", FT, TN)
    k4 = "(ploop 0 %d tile_n n %s)" % (N, _st(
        "tensor", "O_FF", "(+ %s (/ %s (bcast (sqrt (/ %s %d)) 1)))" % (_ld("tensor", "FF2", FT, TN), a2n, o3, N), FT, TN))
    offk = _ld("tensor", "O_FF", FT, TK)
    k5 = _seq("(sloop 0 %d tile_k k %s)" % (N, _st("tensor", "O_FF1", "(+ (x %s 1) (rsum (sqr %s) 1))" % (
        _ld("tensor", "O_FF1", FT), offk), FT)),
        "(ploop 0 %d tile_n n %s)" % (N, _st("output", "O_FF_norm", "(/ %s (bcast (sqrt (/ %s %d)) 1))" % (
            _ld("tensor", "O_FF", FT, TN), _ld("tensor", "O_FF1", FT), N), FT, TN)))
    return _seq(k1, k2, k3, k4, k5)


def rmsnorm_ir(N):
    """Standalone RMSNorm: sum of squares over the row, then the scaled row."""
    k1 = "(sloop 0 %d tile_k k %s)" % (N, _st("tensor", "O_FF1", "(+ (x %s 1) (rsum (sqr %s) 1))" % (
        _ld("tensor", "O_FF1", FT), _ld("input", "O_FF", FT, TK)), FT))
    k2 = "(ploop 0 %d tile_k k %s)" % (N, _st("output", "O_FF_norm", "(/ %s (bcast (sqrt (/ %s %d)) 1))" % (
        _ld("input", "O_FF", FT, TK), _ld("tensor", "O_FF1", FT), N), FT, TK))
    return _seq(k1, k2)
