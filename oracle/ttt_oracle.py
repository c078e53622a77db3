"""CPU oracle for the fused TTT inner loop -- TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the arithmetic of the reference's Burn-op inner
models (the path the reference itself treats as ground truth).  It is the checker
for the HIP kernels: only the test-suite, the smoke check and the benchmark's
`cpu_baseline` leg may import it.  Nothing under the product package calls it.

Each function cites the reference lines it follows (paths relative to the
reference checkout):

  ln_fwd              rust/core/src/util.rs:141-150   (reference/ttt.py:461-475)
  ln_l2_grad          rust/core/src/util.rs:155-182   (reference/ttt.py:478-505)
  gelu_tanh           rust/thundercube/src/unary_ops.rs:136-150
  gelu_tanh_bwd       rust/thundercube/src/unary_ops.rs:152-173 (reference/ttt.py:509-512)
  linear_mini_batch   rust/core/src/linear.rs:91-149
  linear_forward      rust/core/src/inner.rs:25-50 + checkpoints as
                      rust/fused/src/linear_fused_tile/forward/kernel.rs:143-150
  linear_backward     rust/fused/src/linear_fused_tile/backward/kernel.rs:253-429,
                      backward/stage.rs:42-1006, layer_norm.rs:428-709
  mlp_mini_batch      rust/core/src/mlp.rs:127-208
  mlp_forward         rust/core/src/inner.rs:25-50
  mlpn_mini_batch, mlpn_forward
                      rust/core/src/mlp2.rs:152-243, mlp3.rs:162-279, mlp4.rs:186-324 (2, 3, 4 hidden layers)
  linear_adam_mini_batch, linear_adam_forward
                      rust/core/src/linear_adam.rs:76-128 (adam_update), :183-236 (forward_mini_batch)

How each function is pinned (tests/test_oracle_*.py):
  ln_fwd            == torch.nn.functional.layer_norm (library routine)
  ln_l2_grad        == torch autograd of 0.5*||LN(x)-T||^2 w.r.t. x
  gelu_tanh[_bwd]   == torch gelu(approximate="tanh") and its autograd
  linear_mini_batch == primal per-token gradient descent written independently
                       in the test (dual form == primal form invariant), plus the
                       lr==0 and constant-row closed forms
  linear_forward    == chaining single mini-batch calls; checkpoint c == state
                       entering stage c*ci
  linear_backward   == torch autograd (float64) through the independent primal
                       formulation, plus central finite differences of
                       linear_forward
  mlp_mini_batch    == primal per-token GD on both layers, written in the test
  mlp_backward      == torch autograd (float64, double backward) through a torch restatement of the dual
                       form whose forward is checked against mlp_forward, plus linearity
  mlpn_*            == mlp_mini_batch for one hidden layer; primal per-token GD on all layers (autograd through the
                       network, written in the test) for two and three
  linear_adam_*     == the gradients of linear_mini_batch fed to torch.optim.Adam (library routine) step by step;
                       first step from zero moments moves every element by lr*g/(|g|+eps) (closed form);
                       output of a mini-batch == linear_mini_batch's (the output does not see the update)
  lr_logit_grad     == central finite differences of linear_forward through the gate
  rope_apply        == complex rotation of adjacent pairs; inner_loop_inputs, layer_epilogue == their pieces
                       (torch sigmoid / layer_norm / gelu) assembled independently in the test
Frozen results of these functions for five small cases are kept in tests/golden (written by
tests/golden/make_fixtures.py); tests/test_golden_cpu.py holds this module to them.
The reference commits no golden vectors for this path (its fixtures are generated
at test time), so absolute agreement with Burn-CPU's floating-point results is
"parity unpinned"; agreement is to tolerance against this float64 restatement.
"""
from __future__ import annotations

import numpy as np

GELU_C = 0.7978845608028654  # sqrt(2/pi); reference uses 0.79788456 (unary_ops.rs:136)
GELU_A = 0.044715


# --------------------------------------------------------------------------- LayerNorm
def ln_fwd(x, gamma, beta, eps=1e-6):
    """util.rs:141-150. Biased variance, eps inside the sqrt. gamma/beta broadcast on last dim."""
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    std = np.sqrt(var + eps)
    return gamma * ((x - mu) / std) + beta


def ln_l2_grad(x, target, gamma, beta, eps=1e-6):
    """util.rs:155-182. Returns d/dx 0.5*||LN(x)-target||^2."""
    d = x.shape[-1]
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    std = np.sqrt(var + eps)
    xhat = (x - mu) / std
    out = gamma * xhat + beta
    dl_dout = out - target
    dl_dnorm = dl_dout * gamma
    t1 = dl_dnorm * d
    t2 = dl_dnorm.sum(-1, keepdims=True)
    t3 = xhat * (dl_dnorm * xhat).sum(-1, keepdims=True)
    return (t1 - t2 - t3) / (std * d)


# --------------------------------------------------------------------------- GELU
def gelu_tanh(x):
    """unary_ops.rs:136-150."""
    return 0.5 * x * (1.0 + np.tanh(GELU_C * (x + GELU_A * x ** 3)))


def gelu_tanh_bwd(x):
    """unary_ops.rs:152-173; ttt.py:509-512."""
    t = np.tanh(GELU_C * (x + GELU_A * x ** 3))
    return 0.5 * (1.0 + t) + 0.5 * x * (1.0 - t * t) * GELU_C * (1.0 + 3.0 * GELU_A * x * x)


def gelu_tanh_bwd2(x):
    """Second derivative of the tanh-GELU (unary_ops.rs:175-195), needed by the TTT-MLP backward.
    With u = c (x + a x^3), t = tanh u, u' = c (1 + 3 a x^2), u'' = 6 a c x:
    gelu'' = (1 - t^2) u' + 0.5 x (1 - t^2) (u'' - 2 t u'^2)."""
    t = np.tanh(GELU_C * (x + GELU_A * x ** 3))
    du = GELU_C * (1.0 + 3.0 * GELU_A * x * x)
    ddu = 6.0 * GELU_A * GELU_C * x
    s = 1.0 - t * t
    return s * du + 0.5 * x * s * (ddu - 2.0 * t * du * du)


# --------------------------------------------------------------------------- helpers
def _hb(p):
    """[H,d] parameter -> broadcastable [1,H,1,d]."""
    return p[None, :, None, :]


def _eta(token_eta, lr):
    """linear.rs:111-117: eta[i,j] = token_eta[i]*lr[j], lower triangular. lr [B,H,K]."""
    k = lr.shape[-1]
    e = token_eta[None, None, :, None] * lr[:, :, None, :]
    return e * np.tril(np.ones((k, k), dtype=lr.dtype))


def _T(a):
    return np.swapaxes(a, -1, -2)


# --------------------------------------------------------------------------- TTT-Linear
def linear_mini_batch(W, b, xq, xk, xv, token_eta, lr, gamma, beta, eps=1e-6):
    """linear.rs:91-149. One mini-batch.

    W [B,H,d,d], b [B,H,d], xq/xk/xv [B,H,K,d], token_eta [K], lr [B,H,K], gamma/beta [H,d].
    Returns (out [B,H,K,d], W_new, b_new).
    """
    k = xq.shape[2]
    tri = np.tril(np.ones((k, k), dtype=W.dtype))
    z1 = xk @ W + b[:, :, None, :]                                  # :103
    target = xv - xk                                                # :105
    g = ln_l2_grad(z1, target, _hb(gamma), _hb(beta), eps)          # :107-109
    eta = _eta(token_eta, lr)                                       # :111-117
    attn = (xq @ _T(xk)) * tri                                      # :119-121
    b_bar = b[:, :, None, :] - eta @ g                              # :123-124
    z_bar = xq @ W - (eta * attn) @ g + b_bar                       # :126-128
    last = eta[:, :, -1, :]                                         # :130-132  [B,H,K]
    W_new = W - _T(last[..., None] * xk) @ g                        # :134-138
    b_new = b - (last[..., None] * g).sum(2)                        # :140-144
    out = xq + ln_fwd(z_bar, _hb(gamma), _hb(beta), eps)            # :146-148
    return out, W_new, b_new


def linear_forward(W0, b0, xq, xk, xv, token_eta, lr, gamma, beta, K=16, eps=1e-6,
                   checkpoint_interval=0, dtype=np.float64):
    """inner.rs:25-50: sequential loop over mini-batches; a trailing remainder < K is
    processed as one short mini-batch (inner.rs:40-47).

    W0 [H,d,d] (or [B,H,d,d]), b0 [H,d] (or [B,H,d]); token_eta is either [seq]
    (sliced per mini-batch as inner.rs:123-130) or [K] (position inside the mini-batch).
    If checkpoint_interval > 0 also returns W/b entering every stage c*ci
    (forward/kernel.rs:143-150), shape [B,H,ceil(N/ci),d,d] / [B,H,ceil(N/ci),d].
    """
    xq, xk, xv, lr = (np.asarray(a, dtype=dtype) for a in (xq, xk, xv, lr))
    gamma, beta = np.asarray(gamma, dtype=dtype), np.asarray(beta, dtype=dtype)
    token_eta = np.asarray(token_eta, dtype=dtype)
    B, H, seq, d = xq.shape
    W = np.asarray(W0, dtype=dtype)
    b = np.asarray(b0, dtype=dtype)
    if W.ndim == 3:                                                 # init_state, linear.rs:84-89
        W = np.broadcast_to(W[None], (B, H, d, d)).copy()
        b = np.broadcast_to(b[None], (B, H, d)).copy()
    out = np.zeros_like(xq)
    Wc, bc = [], []
    stage = 0
    for s0 in range(0, seq, K):
        s1 = min(s0 + K, seq)
        if checkpoint_interval and stage % checkpoint_interval == 0:
            Wc.append(W.copy())
            bc.append(b.copy())
        te = token_eta[s0:s1] if token_eta.shape[0] == seq and seq != K else token_eta[: s1 - s0]
        o, W, b = linear_mini_batch(W, b, xq[:, :, s0:s1], xk[:, :, s0:s1], xv[:, :, s0:s1],
                                    te, lr[:, :, s0:s1], gamma, beta, eps)
        out[:, :, s0:s1] = o
        stage += 1
    if checkpoint_interval:
        return out, W, b, np.stack(Wc, 2), np.stack(bc, 2)
    return out, W, b


# --------------------------------------------------------------------------- TTT-MLP with several hidden layers
def mlpn_mini_batch(Ws, bs, xq, xk, xv, token_eta, lr, gamma, beta, eps=1e-6):
    """mlp2.rs:152-243 (two hidden layers), mlp3.rs:162-279 (three), mlp4.rs:186-324 (four); with one hidden layer it is
    mlp.rs:127-208.  Ws[i] [B,H,in_i,out_i], bs[i] [B,H,out_i] for the n+1 weight layers d -> 4d -> ... -> 4d -> d.
    Returns (out, new Ws, new bs)."""
    n = len(Ws) - 1                                                 # hidden layers
    k = xq.shape[2]
    tri = np.tril(np.ones((k, k), dtype=xq.dtype))
    x, z = [xk], []                                                 # x[i]: input of weight layer i
    for i in range(n):                                              # mlp2.rs:162-168
        z.append(x[i] @ Ws[i] + bs[i][:, :, None, :])
        x.append(gelu_tanh(z[i]))
    z.append(x[n] @ Ws[n] + bs[n][:, :, None, :])                   # :170
    g = [None] * (n + 1)
    g[n] = ln_l2_grad(z[n], xv - xk, _hb(gamma), _hb(beta), eps)    # :172-176
    for i in range(n - 1, -1, -1):                                  # :178-182
        g[i] = (g[i + 1] @ _T(Ws[i + 1])) * gelu_tanh_bwd(z[i])
    eta = _eta(token_eta, lr)                                       # :184-187
    xb = xq
    for i in range(n + 1):                                          # :189-211
        attn = (xb @ _T(x[i])) * tri
        zb = xb @ Ws[i] - (eta * attn) @ g[i] + (bs[i][:, :, None, :] - eta @ g[i])
        xb = gelu_tanh(zb) if i < n else zb
    last = eta[:, :, -1, :]                                         # :213-214
    Wn = [Ws[i] - _T(last[..., None] * x[i]) @ g[i] for i in range(n + 1)]   # :216-238
    bn = [bs[i] - (last[..., None] * g[i]).sum(2) for i in range(n + 1)]
    return xq + ln_fwd(xb, _hb(gamma), _hb(beta), eps), Wn, bn      # :240-242


def mlpn_forward(Ws0, bs0, xq, xk, xv, token_eta, lr, gamma, beta, K=16, eps=1e-6, dtype=np.float64):
    """inner.rs:25-50 over mlpn_mini_batch.  Ws0[i] [H,in,out] (or [B,H,in,out]); returns (out, Ws, bs)."""
    xq, xk, xv, lr = (np.asarray(a, dtype=dtype) for a in (xq, xk, xv, lr))
    gamma, beta = np.asarray(gamma, dtype=dtype), np.asarray(beta, dtype=dtype)
    token_eta = np.asarray(token_eta, dtype=dtype)
    B, H, seq, d = xq.shape
    Ws = [np.asarray(a, dtype=dtype) for a in Ws0]
    bs = [np.asarray(a, dtype=dtype) for a in bs0]
    if Ws[0].ndim == 3:
        Ws = [np.broadcast_to(a[None], (B,) + a.shape).copy() for a in Ws]
        bs = [np.broadcast_to(a[None], (B,) + a.shape).copy() for a in bs]
    out = np.zeros_like(xq)
    for s0 in range(0, seq, K):
        s1 = min(s0 + K, seq)
        te = token_eta[s0:s1] if token_eta.shape[0] == seq and seq != K else token_eta[: s1 - s0]
        o, Ws, bs = mlpn_mini_batch(Ws, bs, xq[:, :, s0:s1], xk[:, :, s0:s1], xv[:, :, s0:s1], te, lr[:, :, s0:s1],
                                    gamma, beta, eps)
        out[:, :, s0:s1] = o
    return out, Ws, bs


# --------------------------------------------------------------------------- TTT-Linear with an Adam inner optimiser
def linear_adam_mini_batch(state, xq, xk, xv, token_eta, lr, gamma, beta, eps=1e-6, beta1=0.9, beta2=0.999,
                           adam_eps=1e-8, adam_lr=1e-3):
    """linear_adam.rs:183-236: the mini-batch of TTT-Linear with the state update replaced by one Adam step on the
    same eta-weighted gradients (adam_update, linear_adam.rs:76-128).  state = dict(W, b, Wm, bm, Wv, bv, step);
    returns (out, new state).  The output is computed from the state entering the mini-batch, as in linear.rs."""
    W, b = state["W"], state["b"]
    k = xq.shape[2]
    tri = np.tril(np.ones((k, k), dtype=W.dtype))
    z1 = xk @ W + b[:, :, None, :]                                  # :196
    g = ln_l2_grad(z1, xv - xk, _hb(gamma), _hb(beta), eps)         # :198-202
    eta = _eta(token_eta, lr)                                       # :204-208
    attn = (xq @ _T(xk)) * tri                                      # :210
    b_bar = b[:, :, None, :] - eta @ g                              # :212-213
    z_bar = xq @ W - (eta * attn) @ g + b_bar                       # :215-217
    last = eta[:, :, -1, :]                                         # :219-220
    gW = _T(last[..., None] * xk) @ g                               # :222-224
    gb = (last[..., None] * g).sum(2)                               # :226-228
    step = state["step"] + 1                                        # :91
    Wm = state["Wm"] * beta1 + gW * (1.0 - beta1)                   # :102-103
    bm = state["bm"] * beta1 + gb * (1.0 - beta1)
    Wv = state["Wv"] * beta2 + gW ** 2 * (1.0 - beta2)              # :106-111
    bv = state["bv"] * beta2 + gb ** 2 * (1.0 - beta2)
    c1, c2 = 1.0 - beta1 ** step, 1.0 - beta2 ** step               # :113-114
    W_new = W - (Wm / c1) / (np.sqrt(Wv / c2) + adam_eps) * adam_lr  # :116-126
    b_new = b - (bm / c1) / (np.sqrt(bv / c2) + adam_eps) * adam_lr
    out = xq + ln_fwd(z_bar, _hb(gamma), _hb(beta), eps)            # :232-234
    return out, dict(W=W_new, b=b_new, Wm=Wm, bm=bm, Wv=Wv, bv=bv, step=step)


def linear_adam_forward(W0, b0, xq, xk, xv, token_eta, lr, gamma, beta, K=16, eps=1e-6, beta1=0.9, beta2=0.999,
                        adam_eps=1e-8, adam_lr=1e-3, state0=None, dtype=np.float64):
    """inner.rs:25-50 over linear_adam_mini_batch; the state starts with zero moments and step 0
    (init_state, linear_adam.rs:164-177) unless state0 = dict(Wm, bm, Wv, bv, step) continues an earlier call.
    Returns (out, final state dict)."""
    xq, xk, xv, lr = (np.asarray(a, dtype=dtype) for a in (xq, xk, xv, lr))
    gamma, beta = np.asarray(gamma, dtype=dtype), np.asarray(beta, dtype=dtype)
    token_eta = np.asarray(token_eta, dtype=dtype)
    B, H, seq, d = xq.shape
    W, b = np.asarray(W0, dtype=dtype), np.asarray(b0, dtype=dtype)
    if W.ndim == 3:
        W = np.broadcast_to(W[None], (B, H, d, d)).copy()
        b = np.broadcast_to(b[None], (B, H, d)).copy()
    st = dict(W=W, b=b, Wm=np.zeros_like(W), bm=np.zeros_like(b), Wv=np.zeros_like(W), bv=np.zeros_like(b), step=0)
    if state0 is not None:
        st.update({k: (np.asarray(v, dtype=dtype) if k != "step" else int(v)) for k, v in state0.items()})
    out = np.zeros_like(xq)
    for s0 in range(0, seq, K):
        s1 = min(s0 + K, seq)
        te = token_eta[s0:s1] if token_eta.shape[0] == seq and seq != K else token_eta[: s1 - s0]
        o, st = linear_adam_mini_batch(st, xq[:, :, s0:s1], xk[:, :, s0:s1], xv[:, :, s0:s1], te, lr[:, :, s0:s1],
                                       gamma, beta, eps, beta1, beta2, adam_eps, adam_lr)
        out[:, :, s0:s1] = o
    return out, st


def _ln_l2_parts(z1, target, gamma, beta, eps):
    d = z1.shape[-1]
    mu = z1.mean(-1, keepdims=True)
    std = np.sqrt(((z1 - mu) ** 2).mean(-1, keepdims=True) + eps)
    xhat = (z1 - mu) / std
    gO = gamma * xhat + beta - target
    gx = gO * gamma
    G = (d * gx - gx.sum(-1, keepdims=True) - xhat * (gx * xhat).sum(-1, keepdims=True)) / (std * d)
    return xhat, std, gO, gx, G


def linear_backward(W0, b0, xq, xk, xv, token_eta, lr, gamma, beta, d_out, K=16, eps=1e-6,
                    d_W_out=None, d_b_out=None, dtype=np.float64):
    """Reverse scan over mini-batches (backward/kernel.rs:334-417) applying the one-stage
    backward (backward/stage.rs:42-1006; second-order LN term layer_norm.rs:428-709).

    seq must be a multiple of K (forward/launch.rs:209-213); token_eta is [K].
    Returns dict with d_xq,d_xk,d_xv [B,H,seq,d]; d_W0 [B,H,d,d]; d_b0 [B,H,d];
    d_lr [B,H,seq]; d_token_eta [seq] (per position, summed over batch and heads,
    backward/kernel.rs:390); d_gamma,d_beta [H,d] (summed over batch; both the output-LN
    and the through-G contributions, backward/stage.rs:991-994).
    Upstream grads of the final state default to zero (launch.rs:188-194).
    """
    xq, xk, xv, lr, d_out = (np.asarray(a, dtype=dtype) for a in (xq, xk, xv, lr, d_out))
    gamma, beta = np.asarray(gamma, dtype=dtype), np.asarray(beta, dtype=dtype)
    te = np.asarray(token_eta, dtype=dtype)
    B, H, seq, d = xq.shape
    assert seq % K == 0 and te.shape[0] == K
    N = seq // K
    W = np.asarray(W0, dtype=dtype)
    b = np.asarray(b0, dtype=dtype)
    if W.ndim == 3:
        W = np.broadcast_to(W[None], (B, H, d, d)).copy()
        b = np.broadcast_to(b[None], (B, H, d)).copy()
    # forward sweep keeping the state entering every stage (checkpoint_interval = 1)
    Ws, bs = [], []
    for t in range(N):
        Ws.append(W)
        bs.append(b)
        sl = slice(t * K, (t + 1) * K)
        _, W, b = linear_mini_batch(W, b, xq[:, :, sl], xk[:, :, sl], xv[:, :, sl], te,
                                    lr[:, :, sl], gamma, beta, eps)
    dW = np.zeros((B, H, d, d), dtype) if d_W_out is None else np.asarray(d_W_out, dtype).copy()
    db = np.zeros((B, H, d), dtype) if d_b_out is None else np.asarray(d_b_out, dtype).copy()
    g_xq, g_xk, g_xv = np.zeros_like(xq), np.zeros_like(xq), np.zeros_like(xq)
    g_lr = np.zeros_like(lr)
    g_te = np.zeros(seq, dtype)
    g_gamma = np.zeros((H, d), dtype)
    g_beta = np.zeros((H, d), dtype)
    gam, bet = _hb(gamma), _hb(beta)
    tri = np.tril(np.ones((K, K), dtype))
    for t in range(N - 1, -1, -1):
        sl = slice(t * K, (t + 1) * K)
        Q, Kk, V, l = xq[:, :, sl], xk[:, :, sl], xv[:, :, sl], lr[:, :, sl]
        W, b = Ws[t], bs[t]
        dO = d_out[:, :, sl]
        # recompute forward intermediates (stage.rs:123-234)
        z1 = Kk @ W + b[:, :, None, :]
        xhat, std, gO, gx, G = _ln_l2_parts(z1, V - Kk, gam, bet, eps)
        eta = _eta(te, l)
        A = (Q @ _T(Kk)) * tri
        zb = Q @ W + b[:, :, None, :] - (eta + eta * A) @ G
        mu2 = zb.mean(-1, keepdims=True)
        std2 = np.sqrt(((zb - mu2) ** 2).mean(-1, keepdims=True) + eps)
        xhat2 = (zb - mu2) / std2
        last = te[K - 1] * l                                         # [B,H,K]
        # stage 4: output LayerNorm backward (stage.rs:240-298)
        g_gamma += (dO * xhat2).sum((0, 2))
        g_beta += dO.sum((0, 2))
        gx2 = dO * gam
        dzb = (d * gx2 - gx2.sum(-1, keepdims=True)
               - xhat2 * (gx2 * xhat2).sum(-1, keepdims=True)) / (d * std2)
        # stage 3: dual-form terms (stage.rs:300-648)
        P = dzb @ _T(G)                                              # [B,H,K,K]
        dA = -(P * eta) * tri
        dQ = dO + dzb @ _T(W) + dA @ Kk
        dK = _T(dA) @ Q - last[..., None] * (G @ _T(dW))
        S = Kk @ dW + db[:, :, None, :]
        dG = -_T(eta + eta * A) @ dzb - last[..., None] * S
        deta = -(P * tri) * (1.0 + A)
        dlast = -(G * S).sum(-1)                                     # [B,H,K]
        dl = (deta * te[None, None, :, None]).sum(2) + te[K - 1] * dlast
        dte = (deta * l[:, :, None, :]).sum(-1)                      # [B,H,K]
        dte[:, :, K - 1] += (dlast * l).sum(-1)
        dW_new = dW + _T(Q) @ dzb
        db_new = db + dzb.sum(2)
        # stage 2: through G, second-order LayerNorm (layer_norm.rs:428-709)
        u = -dG / std
        s1 = u.sum(-1, keepdims=True)
        s2 = (u * xhat).sum(-1, keepdims=True)
        dgx = dG / std + s1 / d + xhat * s2 / d
        dy = gam * dgx
        dT = -dy
        g_gamma += (gO * dgx + dy * xhat).sum((0, 2))
        g_beta += dy.sum((0, 2))
        dxhat = dy * gam + gx * s2 / d + u * (gx * xhat).sum(-1, keepdims=True) / d
        dstd = (-(dxhat * xhat + dG * G) / std).sum(-1, keepdims=True)
        dz1 = dxhat / std - dxhat.sum(-1, keepdims=True) / (d * std) + xhat * dstd / d
        # stage 1: matmul backward (stage.rs:933-988)
        g_xq[:, :, sl] = dQ
        g_xv[:, :, sl] = dT
        g_xk[:, :, sl] = dK - dT + dz1 @ _T(W)
        dW = dW_new + _T(Kk) @ dz1
        db = db_new + dz1.sum(2)
        g_lr[:, :, sl] = dl
        g_te[sl] = dte.sum((0, 1))
    return dict(d_xq=g_xq, d_xk=g_xk, d_xv=g_xv, d_W0=dW, d_b0=db, d_lr=g_lr,
                d_token_eta=g_te, d_gamma=g_gamma, d_beta=g_beta)


# --------------------------------------------------------------------------- TTT-MLP
def mlp_mini_batch(W1, b1, W2, b2, xq, xk, xv, token_eta, lr, gamma, beta, eps=1e-6):
    """mlp.rs:127-208. W1 [B,H,d,4d], b1 [B,H,4d], W2 [B,H,4d,d], b2 [B,H,d]."""
    k = xq.shape[2]
    tri = np.tril(np.ones((k, k), dtype=W1.dtype))
    z1 = xk @ W1 + b1[:, :, None, :]                                # :139
    x2 = gelu_tanh(z1)                                              # :141
    z2 = x2 @ W2 + b2[:, :, None, :]                                # :143
    target = xv - xk                                                # :145
    g2 = ln_l2_grad(z2, target, _hb(gamma), _hb(beta), eps)         # :147-149
    g1 = (g2 @ _T(W2)) * gelu_tanh_bwd(z1)                          # :151-152
    eta = _eta(token_eta, lr)                                       # :154-158
    attn1 = (xq @ _T(xk)) * tri                                     # :160-162
    b1_bar = b1[:, :, None, :] - eta @ g1                           # :164-165
    z1_bar = xq @ W1 - (eta * attn1) @ g1 + b1_bar                  # :167-169
    x2_bar = gelu_tanh(z1_bar)                                      # :171
    attn2 = (x2_bar @ _T(x2)) * tri                                 # :173
    b2_bar = b2[:, :, None, :] - eta @ g2                           # :175-176
    z2_bar = x2_bar @ W2 - (eta * attn2) @ g2 + b2_bar              # :178-180
    last = eta[:, :, -1, :]                                         # :182-183
    W1n = W1 - _T(last[..., None] * xk) @ g1                        # :185-188
    b1n = b1 - (last[..., None] * g1).sum(2)                        # :190-193
    W2n = W2 - _T(last[..., None] * x2) @ g2                        # :195-198
    b2n = b2 - (last[..., None] * g2).sum(2)                        # :200-203
    out = xq + ln_fwd(z2_bar, _hb(gamma), _hb(beta), eps)           # :205-207
    return out, W1n, b1n, W2n, b2n


def mlp_forward(W1_0, b1_0, W2_0, b2_0, xq, xk, xv, token_eta, lr, gamma, beta, K=16,
                eps=1e-6, dtype=np.float64):
    """inner.rs:25-50 over mlp_mini_batch. Initial state [H,...] is broadcast over batch
    (mlp.rs:119-125). Returns (out, W1, b1, W2, b2)."""
    xq, xk, xv, lr = (np.asarray(a, dtype=dtype) for a in (xq, xk, xv, lr))
    gamma, beta = np.asarray(gamma, dtype=dtype), np.asarray(beta, dtype=dtype)
    token_eta = np.asarray(token_eta, dtype=dtype)
    B, H, seq, d = xq.shape
    st = [np.asarray(a, dtype=dtype) for a in (W1_0, b1_0, W2_0, b2_0)]
    if st[0].ndim == 3:
        st = [np.broadcast_to(a[None], (B,) + a.shape).copy() for a in st]
    out = np.zeros_like(xq)
    for s0 in range(0, seq, K):
        s1 = min(s0 + K, seq)
        te = token_eta[s0:s1] if token_eta.shape[0] == seq and seq != K else token_eta[: s1 - s0]
        o, *st = mlp_mini_batch(*st, xq[:, :, s0:s1], xk[:, :, s0:s1], xv[:, :, s0:s1],
                                te, lr[:, :, s0:s1], gamma, beta, eps)
        out[:, :, s0:s1] = o
    return (out, *st)


def _ln_l2_second_order(dG, xhat, std, gO, gx, G, gam, d):
    """Backward of G = ln_l2_grad(z, T) given dG (layer_norm.rs:428-709): returns dz, dT and the
    [B,H,K,d] summands of d_gamma, d_beta."""
    u = -dG / std
    s1 = u.sum(-1, keepdims=True)
    s2 = (u * xhat).sum(-1, keepdims=True)
    dgx = dG / std + s1 / d + xhat * s2 / d
    dy = gam * dgx
    dxhat = dy * gam + gx * s2 / d + u * (gx * xhat).sum(-1, keepdims=True) / d
    dstd = (-(dxhat * xhat + dG * G) / std).sum(-1, keepdims=True)
    dz = dxhat / std - dxhat.sum(-1, keepdims=True) / (d * std) + xhat * dstd / d
    return dz, -dy, gO * dgx + dy * xhat, dy


def mlp_backward(W1_0, b1_0, W2_0, b2_0, xq, xk, xv, token_eta, lr, gamma, beta, d_out, K=16,
                 eps=1e-6, d_state_out=None, dtype=np.float64):
    """Reverse scan of the TTT-MLP inner loop: the gradient of sum(out * d_out) (plus the inner
    product of the final state with d_state_out = (dW1, db1, dW2, db2), if given) through
    mlp_mini_batch (mlp.rs:127-208) looped as inner.rs:25-50.  The reference has no fused MLP
    backward; it differentiates these ops with Burn autodiff, which this restates in closed form.

    seq must be a multiple of K; token_eta is [K].  Returns a dict: d_xq,d_xk,d_xv [B,H,seq,d];
    d_W1 [B,H,d,4d], d_b1 [B,H,4d], d_W2 [B,H,4d,d], d_b2 [B,H,d] (per batch: the parameter grads are
    their batch sums); d_lr [B,H,seq]; d_token_eta [seq] (per position, summed over batch and
    heads); d_gamma, d_beta [H,d] (summed over batch).
    """
    xq, xk, xv, lr, d_out = (np.asarray(a, dtype=dtype) for a in (xq, xk, xv, lr, d_out))
    gamma, beta = np.asarray(gamma, dtype=dtype), np.asarray(beta, dtype=dtype)
    te = np.asarray(token_eta, dtype=dtype)
    B, H, seq, d = xq.shape
    assert seq % K == 0 and te.shape[0] == K
    N = seq // K
    st = [np.asarray(a, dtype=dtype) for a in (W1_0, b1_0, W2_0, b2_0)]
    if st[0].ndim == 3:
        st = [np.broadcast_to(a[None], (B,) + a.shape).copy() for a in st]
    states = []
    for t in range(N):
        states.append(st)
        sl = slice(t * K, (t + 1) * K)
        _, *st = mlp_mini_batch(*st, xq[:, :, sl], xk[:, :, sl], xv[:, :, sl], te, lr[:, :, sl],
                                gamma, beta, eps)
    if d_state_out is None:
        dW1, db1, dW2, db2 = (np.zeros_like(a) for a in st)
    else:
        dW1, db1, dW2, db2 = (np.asarray(a, dtype).copy() for a in d_state_out)
    g_xq, g_xk, g_xv = np.zeros_like(xq), np.zeros_like(xq), np.zeros_like(xq)
    g_lr = np.zeros_like(lr)
    g_te = np.zeros(seq, dtype)
    g_gamma = np.zeros((H, d), dtype)
    g_beta = np.zeros((H, d), dtype)
    gam, bet = _hb(gamma), _hb(beta)
    tri = np.tril(np.ones((K, K), dtype))
    for t in range(N - 1, -1, -1):
        sl = slice(t * K, (t + 1) * K)
        Q, Kk, V, l = xq[:, :, sl], xk[:, :, sl], xv[:, :, sl], lr[:, :, sl]
        W1, b1, W2, b2 = states[t]
        dO = d_out[:, :, sl]
        # ---- forward intermediates of this mini-batch (mlp.rs:139-183)
        z1 = Kk @ W1 + b1[:, :, None, :]
        x2, ph1 = gelu_tanh(z1), gelu_tanh_bwd(z1)
        z2 = x2 @ W2 + b2[:, :, None, :]
        xhat, std, gO, gx, G2 = _ln_l2_parts(z2, V - Kk, gam, bet, eps)
        U = G2 @ _T(W2)
        G1 = U * ph1
        eta = _eta(te, l)
        A1 = (Q @ _T(Kk)) * tri
        z1b = Q @ W1 + b1[:, :, None, :] - (eta + eta * A1) @ G1
        x2b, ph1b = gelu_tanh(z1b), gelu_tanh_bwd(z1b)
        A2 = (x2b @ _T(x2)) * tri
        z2b = x2b @ W2 + b2[:, :, None, :] - (eta + eta * A2) @ G2
        mu2 = z2b.mean(-1, keepdims=True)
        std2 = np.sqrt(((z2b - mu2) ** 2).mean(-1, keepdims=True) + eps)
        xhat2 = (z2b - mu2) / std2
        last = te[K - 1] * l
        # ---- output LayerNorm
        g_gamma += (dO * xhat2).sum((0, 2))
        g_beta += dO.sum((0, 2))
        gx2 = dO * gam
        dz2b = (d * gx2 - gx2.sum(-1, keepdims=True)
                - xhat2 * (gx2 * xhat2).sum(-1, keepdims=True)) / (d * std2)
        # ---- second layer, dual-form terms
        P2 = dz2b @ _T(G2)
        dA2 = -(P2 * eta) * tri
        deta = -(P2 * tri) * (1.0 + A2)
        dx2b = dz2b @ _T(W2) + dA2 @ x2
        dx2 = _T(dA2) @ x2b - last[..., None] * (G2 @ _T(dW2))
        S2 = x2 @ dW2 + db2[:, :, None, :]
        dG2 = -_T(eta + eta * A2) @ dz2b - last[..., None] * S2
        dlast = -(G2 * S2).sum(-1)
        # ---- first layer, dual-form terms
        dz1b = dx2b * ph1b
        P1 = dz1b @ _T(G1)
        dA1 = -(P1 * eta) * tri
        deta += -(P1 * tri) * (1.0 + A1)
        dQ = dO + dz1b @ _T(W1) + dA1 @ Kk
        dK = _T(dA1) @ Q - last[..., None] * (G1 @ _T(dW1))
        S1 = Kk @ dW1 + db1[:, :, None, :]
        dG1 = -_T(eta + eta * A1) @ dz1b - last[..., None] * S1
        dlast += -(G1 * S1).sum(-1)
        # ---- G1 = (G2 W2^T) * gelu'(z1)
        dU = dG1 * ph1
        dG2 = dG2 + dU @ W2
        # ---- G2 = LN-L2 gradient of z2: second-order LayerNorm
        dz2, dT, sg, sb = _ln_l2_second_order(dG2, xhat, std, gO, gx, G2, gam, d)
        g_gamma += sg.sum((0, 2))
        g_beta += sb.sum((0, 2))
        dx2 = dx2 + dz2 @ _T(W2)
        dz1 = dG1 * U * gelu_tanh_bwd2(z1) + dx2 * ph1
        # ---- parameter and input gradients
        dW2 = dW2 + _T(x2b) @ dz2b + _T(dU) @ G2 + _T(x2) @ dz2
        db2 = db2 + dz2b.sum(2) + dz2.sum(2)
        dW1 = dW1 + _T(Q) @ dz1b + _T(Kk) @ dz1
        db1 = db1 + dz1b.sum(2) + dz1.sum(2)
        g_xq[:, :, sl] = dQ
        g_xv[:, :, sl] = dT
        g_xk[:, :, sl] = dK - dT + dz1 @ _T(W1)
        dl = (deta * te[None, None, :, None]).sum(2) + te[K - 1] * dlast
        dte = (deta * l[:, :, None, :]).sum(-1)
        dte[:, :, K - 1] += (dlast * l).sum(-1)
        g_lr[:, :, sl] = dl
        g_te[sl] = dte.sum((0, 1))
    return dict(d_xq=g_xq, d_xk=g_xk, d_xv=g_xv, d_W1=dW1, d_b1=db1, d_W2=dW2, d_b2=db2,
                d_lr=g_lr, d_token_eta=g_te, d_gamma=g_gamma, d_beta=g_beta)


# --------------------------------------------------------------------------- either side of the inner loop
def rope_cos_sin(seq, offset, wrap, head_dim, base=10000.0):
    """RotaryEmbeddingConfig::init + get_cos_sin (util.rs:266-322): inv_freq[i] = 1/base^(2i/d) rounded
    to f32, positions (offset + t), taken modulo `wrap` when given, freqs = pos * inv_freq formed in
    f32 as the reference's backend does; returns (cos, sin) [seq, d/2] (the reference concatenates
    the half twice to [seq, d])."""
    half = head_dim // 2
    inv_freq = np.array([np.float32(1.0 / base ** ((2 * i) / head_dim)) for i in range(half)], np.float32)
    pos = np.arange(seq, dtype=np.float32) + np.float32(offset)
    if wrap is not None:
        pos = np.fmod(pos, np.float32(wrap))
    freqs = (pos[:, None] * inv_freq[None, :]).astype(np.float32).astype(np.float64)
    return np.cos(freqs), np.sin(freqs)


def _permute_qk(x):
    """ttt.rs:26-32: [..., d] -> [..., d/2, 2] -> swap -> [..., 2, d/2] -> [..., d]."""
    s = x.shape
    return np.swapaxes(x.reshape(s[:-1] + (s[-1] // 2, 2)), -1, -2).reshape(s)


def _undo_permute_qk(x):
    """ttt.rs:35-41."""
    s = x.shape
    return np.swapaxes(x.reshape(s[:-1] + (2, s[-1] // 2)), -1, -2).reshape(s)


def _rotate_half(x):
    """util.rs:349-364: [x1, x2] -> [-x2, x1]."""
    h = x.shape[-1] // 2
    return np.concatenate([-x[..., h:], x[..., :h]], -1)


def rope_apply(x, cos, sin):
    """permute_qk -> x*cos + rotate_half(x)*sin -> undo_permute_qk (ttt.rs:179-194,
    util.rs:385-392).  x [B,H,seq,d]; cos/sin [seq, d/2]."""
    c = np.concatenate([cos, cos], -1)[None, None]
    s = np.concatenate([sin, sin], -1)[None, None]
    y = _permute_qk(x)
    return _undo_permute_qk(y * c + _rotate_half(y) * s)


def inner_loop_inputs(xq, xk, xv, lr_logits, lr_bias, base_lr, token_idx, learnable_token_idx, K,
                      cos=None, sin=None, dtype=np.float64):
    """TTT::get_inner_loop_inputs after the projections (ttt.rs:147-194, 205-227, 247-268).
    xq,xk,xv [B,seq,H,d] as the projections (and convolutions) leave them; lr_logits [B,seq,H] =
    x @ learnable_ttt_lr_weight^T.  Returns xq,xk,xv [B,H,seq,d] (RoPE on xq,xk when cos/sin
    [seq,d/2] are given), ttt_lr_eta [B,H,seq], token_eta [seq]."""
    xq, xk, xv, lg = (np.asarray(a, dtype) for a in (xq, xk, xv, lr_logits))
    B, seq, H, d = xq.shape
    q, k, v = (np.transpose(a, (0, 2, 1, 3)) for a in (xq, xk, xv))
    if cos is not None:
        q, k = rope_apply(q, cos, sin), rope_apply(k, cos, sin)
    z = lg + np.asarray(lr_bias, dtype)[None, None, :]
    lr = base_lr * (1.0 / (1.0 + np.exp(-np.transpose(z, (0, 2, 1))))) / d
    te = np.asarray(token_idx, dtype) + np.asarray(learnable_token_idx, dtype)
    te = np.maximum(np.tile(te, -(-seq // K))[:seq], 0.0)
    return q, k, v, lr, te


def lr_logit_grad(d_lr, lr_logits, base_lr, head_dim, dtype=np.float64):
    """Gradient w.r.t. the lr-gate logits from the gradient w.r.t. ttt_lr_eta: the chain through
    ttt_lr_eta = base_lr * sigmoid(logit) / head_dim (get_lr, ttt.rs:205-227).  d_lr and lr_logits have the same
    shape ([B,H,seq]); the gate's bias is part of the logit."""
    g, z = np.asarray(d_lr, dtype), np.asarray(lr_logits, dtype)
    s = 1.0 / (1.0 + np.exp(-z))
    return g * (base_lr / head_dim) * s * (1.0 - s)


def layer_epilogue(inner_out, post_gamma, post_beta, gate=None, eps=1e-6):
    """TTT::forward after the inner model (ttt.rs:285-297): [B,H,seq,d] -> [B,seq,H*d], post_norm
    LayerNorm over the hidden axis (eps 1e-6), times gelu_tanh(gate) when the gate projection exists.
    The output projection that follows is a plain GEMM and not part of this."""
    x = np.asarray(inner_out, np.float64)
    B, H, seq, d = x.shape
    y = ln_fwd(np.transpose(x, (0, 2, 1, 3)).reshape(B, seq, H * d), np.asarray(post_gamma, np.float64),
               np.asarray(post_beta, np.float64), eps)
    return y if gate is None else gelu_tanh(np.asarray(gate, np.float64)) * y
