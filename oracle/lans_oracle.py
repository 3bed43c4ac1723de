"""CPU restatement (NumPy) of the reference's fused multi-tensor LANS step.

TEST INFRASTRUCTURE ONLY (see moe_oracle.py).  Follows
src/op/dialect/cuda/kernels/multi_tensor_lans.cu (L2NormFunctor :95-167, cleanup
:169-185, LANSStage1Functor :207-322, LANSStage2Functor :326-399, driver
:401-450) and src/op/dialect/cuda/lans.cc:92-148 (bias corrections, beta3, list
order [g.. | p.. | m.. | v..]).

The reference's own test oracle is apex.optimizers.FusedLANS
(tests/python/optim/test_lans.py:18-21), which is not in the tree and not
installed, and the tree holds no golden vectors for LANS.  The restatement is
therefore pinned by: the closed form evaluated by hand on a 1-element tensor,
the special cases the formula fixes (norm == 0 -> ratio = lr; beta1 = 0 and
normalize_grad = 0 collapse u_m == u_g; weight_decay = 0 never reads p in
stage 1), an independent fp64 re-derivation written from the LANS paper
(arXiv 2006.13484, Alg. 2) in tests/test_oracle_lans.py, and scale invariance
of the normalised-gradient path.

One deliberate difference from the reference: the reference lays the scratch
`q` buffers (u_g) at offsets numels[i-1] instead of a running sum
(lans.cc:126-129), so they overlap for three or more tensors.  That is a bug,
not semantics; this restatement (like apex) keeps u_g per tensor.

Elementwise math is fp32 in the reference's operation order; the per-tensor
norms are sqrt of an fp64 sum of fp32 squares, rounded to fp32 (the reference
sums fp32 partials in a launch-dependent tree order, which no CPU restatement
can reproduce bit for bit).
"""
import numpy as np

f32 = np.float32


def l2norm(x):
    """multi_tensor_lans.cu:95-185: sqrt(sum x^2) per tensor."""
    x = np.asarray(x, dtype=np.float32).ravel()
    sq = (x * x).astype(np.float32)          # fp32 square, as vals[ii] += next*next
    return f32(np.sqrt(np.sum(sq, dtype=np.float64)))


def bias_corrections(step, beta1, beta2, bias_correction):
    """lans.cc:108-113 (std::pow on float arguments, result stored in float)."""
    if bias_correction:
        return f32(1.0 - float(f32(beta1)) ** int(step)), f32(1.0 - float(f32(beta2)) ** int(step))
    return f32(1.0), f32(1.0)


def lans_step(g_list, p_list, m_list, v_list, step, lr=1e-3, beta1=0.9, beta2=0.999,
              eps=1e-6, bias_correction=1, weight_decay=0.01, grad_averaging=1, mode=1,
              normalize_grad=True):
    """One LANS step over a tensor list, in place on p, m, v (g is left untouched;
    the reference overwrites it with u_m, multi_tensor_lans.cu:314).
    Returns the per-tensor norms (g, p, u_m, u_g) for inspection."""
    beta1, beta2, eps, lr, wd = f32(beta1), f32(beta2), f32(eps), f32(lr), f32(weight_decay)
    bc1, bc2 = bias_corrections(step, beta1, beta2, bias_correction)
    beta3 = f32(1.0) - beta1 if grad_averaging else f32(1.0)     # lans.cc:114-117
    one_minus_b2 = f32(1.0) - beta2
    norms = []
    for g, p, m, v in zip(g_list, p_list, m_list, v_list):
        gn = l2norm(g)                                           # :420
        pn = l2norm(p)                                           # :424
        sg = g.astype(np.float32, copy=True)
        if normalize_grad and gn != 0:                           # :284-286
            sg = sg / (gn + eps)
        rp = p if wd != 0 else np.zeros_like(p)                  # :264-269
        if mode == 0:                                            # :287-297
            sg = sg + wd * rp
        m[...] = m * beta1 + beta3 * sg                          # :290/:299
        v[...] = v * beta2 + one_minus_b2 * sg * sg              # :291/:300
        denom = np.sqrt(v / bc2).astype(np.float32) + eps        # :293-294
        if mode == 0:
            u_m = (m / bc1) / denom
            u_g = sg / denom
        else:                                                    # :304-306
            scaled_p = wd * rp
            u_m = (m / bc1) / denom + scaled_p
            u_g = sg / denom + scaled_p
        umn = l2norm(u_m)                                        # :434
        ugn = l2norm(u_g)                                        # :440
        ratio_m = lr * (pn / umn) if (umn != 0 and pn != 0) else lr   # :349
        ratio_g = lr * (pn / ugn) if (ugn != 0 and pn != 0) else lr   # :350
        ratio_m = f32(ratio_m) * beta1                           # :351
        ratio_g = f32(ratio_g) * beta3                           # :352
        p[...] = p - ratio_m * u_m - ratio_g * u_g               # :386
        norms.append((gn, pn, umn, ugn))
    return norms


def lans_step_mixed(g_list, p_list, m_list, v_list, step, lowp_round=None, **hyper):
    """The step as the reference's traced optimizer runs it for a 16-bit model (python/raf/optim/lans.py:256-257,
    285-288): every gradient cast to float32, lans_step, every new parameter cast back to the model's type.
    g_list holds the 16-bit gradients as the float32 values they denote (the cast is exact); p, m, v are the float32
    master state, updated in place.  Returns the model's copies of the new parameters (float32 values of the 16-bit
    type lowp_round rounds to), or None without lowp_round."""
    lans_step([np.asarray(g, np.float32) for g in g_list], p_list, m_list, v_list, step, **hyper)
    if lowp_round is None:
        return None
    return [lowp_round(p).astype(np.float32) for p in p_list]
