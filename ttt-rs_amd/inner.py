"""Host-side mirror of the reference's inner-model interface for the fused TTT-Linear layer.

Names and argument meaning follow the reference:
  TTTInnerModel trait            rust/core/src/inner.rs:13-58
  Qkv / TTTInputsInner           rust/core/src/inner.rs:60-130
  TTTLinear / TTTLinearState     rust/core/src/linear.rs:17-89
  Fused<_, TTTLinear, TileMultiKernel> ("fused-tile-multi")
                                 rust/fused/src/linear_fused_tile/wrapper.rs:81-211
All arithmetic happens in the HIP library behind include/ttt_mi355x.h.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Optional

import torch

from . import _lib
from ._lib import TttDesc, check, lib


@dataclass
class TTTConfig:
    """Subset of rust/config/src/train.rs:11-141 used by the inner loop."""
    mini_batch_size: int = 16
    base_lr: float = 1.0
    epsilon: float = 1e-6
    checkpoint_interval: int = 1
    mlp_expansion_factor: int = 4


@dataclass
class ModelConfig:
    num_heads: int
    head_dim: int
    ttt: TTTConfig = field(default_factory=TTTConfig)


@dataclass
class Qkv:
    """[batch, heads, seq, head_dim] each (inner.rs:60-68)."""
    xq: torch.Tensor
    xk: torch.Tensor
    xv: torch.Tensor

    def slice_seq(self, r: range) -> "Qkv":
        return Qkv(self.xq[:, :, r.start:r.stop], self.xk[:, :, r.start:r.stop], self.xv[:, :, r.start:r.stop])


@dataclass
class TTTInputsInner:
    """inner.rs:107-119. token_eta [seq] f32, ttt_lr_eta [batch, heads, seq]."""
    qkv: Qkv
    token_eta: torch.Tensor
    ttt_lr_eta: torch.Tensor
    start_idx: int = 0

    def slice_seq(self, r: range) -> "TTTInputsInner":
        return TTTInputsInner(self.qkv.slice_seq(r), self.token_eta[r.start:r.stop],
                              self.ttt_lr_eta[:, :, r.start:r.stop], r.start)


@dataclass
class TTTLinearState:
    """linear.rs:27-33: weight [B,H,d,d], bias [B,H,d], always f32."""
    weight: torch.Tensor
    bias: torch.Tensor


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _io_dtype(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return _lib.TTT_F32
    if t.dtype == torch.bfloat16:
        return _lib.TTT_BF16
    raise _lib.TttError(_lib.TTT_ERR_UNSUPPORTED, f"activation dtype {t.dtype} (f32 or bf16 only)")


def _need(t: torch.Tensor, shape, dtype, name):
    if tuple(t.shape) != tuple(shape):
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, f"{name}: shape {tuple(t.shape)} != {tuple(shape)}")
    if t.dtype != dtype:
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, f"{name}: dtype {t.dtype} != {dtype}")
    if not t.is_cuda:
        raise _lib.TttError(_lib.TTT_ERR_NULL, f"{name} is not a device tensor")
    return t.contiguous()


def _seq_pitch(t: torch.Tensor) -> Optional[int]:
    """Tokens between consecutive (batch, head) units if `t` ([B,H,seq,d] or [B,H,seq]) is a
    window along seq of a dense tensor (what slicing dim 2 of a contiguous tensor gives), else None."""
    trail = t.shape[3] if t.dim() == 4 else 1
    st = t.stride()
    if t.dim() == 4 and (st[3] != 1 or st[2] != trail):
        return None
    if t.dim() == 3 and st[2] != 1:
        return None
    if st[1] % trail or st[0] != t.shape[1] * st[1]:
        return None
    pitch = st[1] // trail
    return pitch if pitch >= t.shape[2] else None


def _common_pitch(seq: int, *tensors) -> int:
    """The shared sequence pitch of the given windows, or 0 when they have to be packed."""
    pitches = {_seq_pitch(t) for t in tensors}
    if len(pitches) == 1 and None not in pitches:
        p = pitches.pop()
        return 0 if p == seq else p
    return 0


def _need_win(t: torch.Tensor, shape, dtype, name, pitch: int):
    """Like _need, but keeps a sequence window in place when a pitch is in use."""
    if pitch == 0:
        return _need(t, shape, dtype, name)
    if tuple(t.shape) != tuple(shape) or t.dtype != dtype or not t.is_cuda:
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, f"{name}: expected {tuple(shape)} {dtype} on the device")
    return t


def ttt_linear_forward_raw(xq, xk, xv, weight, bias, token_eta, ttt_lr_eta, ln_weight, ln_bias,
                           mini_batch: int, eps: float = 1e-6, checkpoint_interval: int = 1,
                           want_checkpoints: bool = False, out: Optional[torch.Tensor] = None, packed_checkpoints: bool = False,
                           kernel_hint: int = 0):
    """One call of ttt_linear_fwd on the current stream.

    Counterpart of fused_ttt_tile_forward_multi (rust/fused/src/linear_fused_tile/api.rs:52-83):
    weight [B,H,d,d] or [H,d,d], bias [B,H,d] or [H,d], token_eta [>=K] (first K entries used).
    Returns (output, weight_out, bias_out[, weight_ckpt, bias_ckpt]).
    packed_checkpoints is ttt_desc.checkpoint_format: False/0 f32 matrices; True/1 (interval 1) W checkpoints as
    operand fragments in kernel order; 2 (bf16 I/O, interval 1, d <= 96) the update factors and the final state
    instead of states.  The result is to be handed to ttt_linear_backward_raw with the same value; the tensors keep
    their f32 [B,H,n,d,d] / [B,H,n,d] allocations whatever the format.
    """
    B, H, seq, d = xq.shape
    io = xq.dtype
    # sequence windows of dense tensors are processed in place (desc.seq_stride) when inputs and
    # the caller's output window share one pitch; anything else is packed first
    pitch = _common_pitch(seq, xq, xk, xv, ttt_lr_eta, out) if out is not None else 0
    xq = _need_win(xq, (B, H, seq, d), io, "xq", pitch)
    xk = _need_win(xk, (B, H, seq, d), io, "xk", pitch)
    xv = _need_win(xv, (B, H, seq, d), io, "xv", pitch)
    lr = _need_win(ttt_lr_eta, (B, H, seq), io, "ttt_lr_eta", pitch)
    per_batch = weight.dim() == 4
    weight = _need(weight, (B, H, d, d) if per_batch else (H, d, d), torch.float32, "weight")
    bias = _need(bias, (B, H, d) if per_batch else (H, d), torch.float32, "bias")
    ln_weight = _need(ln_weight, (H, d), torch.float32, "ln_weight")
    ln_bias = _need(ln_bias, (H, d), torch.float32, "ln_bias")
    if token_eta.numel() < mini_batch:
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, "token_eta shorter than mini_batch")
    te = token_eta.to(torch.float32).contiguous()
    desc = TttDesc(B, H, seq, d, mini_batch, eps, checkpoint_interval, _io_dtype(xq), int(per_batch), pitch,
                   int(packed_checkpoints), kernel_hint)
    check(lib().ttt_linear_supported(C.byref(desc)))
    dev = xq.device
    if out is None or (pitch == 0 and not out.is_contiguous()):
        dst, out = out, torch.empty((B, H, seq, d), dtype=io, device=dev)
    else:
        dst = None
        out = _need_win(out, (B, H, seq, d), io, "out", pitch)
    w_out = torch.empty((B, H, d, d), dtype=torch.float32, device=dev)
    b_out = torch.empty((B, H, d), dtype=torch.float32, device=dev)
    w_ck = b_ck = None
    if want_checkpoints:
        n = lib().ttt_linear_num_checkpoints(C.byref(desc))
        w_ck = torch.empty((B, H, n, d, d), dtype=torch.float32, device=dev)
        b_ck = torch.empty((B, H, n, d), dtype=torch.float32, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    with torch.cuda.device(dev):
        check(lib().ttt_linear_fwd(C.byref(desc), _ptr(xq), _ptr(xk), _ptr(xv), _ptr(weight), _ptr(bias),
                                   _ptr(te), _ptr(lr), _ptr(ln_weight), _ptr(ln_bias), _ptr(out),
                                   _ptr(w_out), _ptr(b_out), _ptr(w_ck), _ptr(b_ck), stream))
    if dst is not None:
        dst.copy_(out)
        out = dst
    if want_checkpoints:
        return out, w_out, b_out, w_ck, b_ck
    return out, w_out, b_out


def ttt_linear_adam_forward_raw(xq, xk, xv, weight, bias, token_eta, ttt_lr_eta, ln_weight, ln_bias, mini_batch: int,
                                beta1: float = 0.9, beta2: float = 0.999, adam_eps: float = 1e-8, adam_lr: float = 1e-3,
                                moments=None, step: int = 0, eps: float = 1e-6):
    """One call of ttt_linear_adam_fwd on the current stream: TTTLinearAdam::forward
    (rust/core/src/linear_adam.rs:183-236 looped as rust/core/src/inner.rs:25-50).  Arguments as
    ttt_linear_forward_raw; moments = (weight_m, bias_m, weight_v, bias_v) per batch element to continue an earlier call
    at `step`, or None for a fresh state.  Returns (output, weight, bias, (weight_m, bias_m, weight_v, bias_v), step)."""
    B, H, seq, d = xq.shape
    io = xq.dtype
    xq = _need(xq, (B, H, seq, d), io, "xq")
    xk = _need(xk, (B, H, seq, d), io, "xk")
    xv = _need(xv, (B, H, seq, d), io, "xv")
    per_batch = weight.dim() == 4
    W0 = _need(weight, (B, H, d, d) if per_batch else (H, d, d), torch.float32, "weight")
    b0 = _need(bias, (B, H, d) if per_batch else (H, d), torch.float32, "bias")
    te = _need(token_eta[:mini_batch], (mini_batch,), torch.float32, "token_eta")
    lr = _need(ttt_lr_eta, (B, H, seq), io, "ttt_lr_eta")
    gam = _need(ln_weight, (H, d), torch.float32, "ln_weight")
    bet = _need(ln_bias, (H, d), torch.float32, "ln_bias")
    dev = xq.device
    f32 = dict(dtype=torch.float32, device=dev)
    null = C.c_void_p(None)
    m_in = [null] * 4
    if moments is not None:
        shapes = ((B, H, d, d), (B, H, d), (B, H, d, d), (B, H, d))
        m_in = [_ptr(_need(t, sh, torch.float32, "moment")) for t, sh in zip(moments, shapes)]
    desc = TttDesc(B, H, seq, d, mini_batch, eps, 1, _io_dtype(xq), 1 if per_batch else 0, 0, 0, 0)
    check(lib().ttt_linear_adam_supported(C.byref(desc)))
    out = torch.empty((B, H, seq, d), dtype=io, device=dev)
    W, b = torch.empty((B, H, d, d), **f32), torch.empty((B, H, d), **f32)
    mo = (torch.empty((B, H, d, d), **f32), torch.empty((B, H, d), **f32), torch.empty((B, H, d, d), **f32),
          torch.empty((B, H, d), **f32))
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    with torch.cuda.device(dev):
        check(lib().ttt_linear_adam_fwd(C.byref(desc), _ptr(xq), _ptr(xk), _ptr(xv), _ptr(W0), _ptr(b0), *m_in, int(step),
                                        C.c_float(beta1), C.c_float(beta2), C.c_float(adam_eps), C.c_float(adam_lr),
                                        _ptr(te), _ptr(lr), _ptr(gam), _ptr(bet), _ptr(out), _ptr(W), _ptr(b),
                                        *[_ptr(t) for t in mo], stream))
    return out, W, b, mo, step + seq // mini_batch


def ttt_linear_backward_raw(xq, xk, xv, weight, bias, token_eta, ttt_lr_eta, ln_weight, ln_bias,
                            weight_ckpt, bias_ckpt, grad_output, mini_batch: int, eps: float = 1e-6,
                            checkpoint_interval: int = 1, grad_weight_out=None, grad_bias_out=None, packed_checkpoints: bool = False,
                            kernel_hint: int = 0, workspace=None):
    """One call of ttt_linear_bwd (or ttt_linear_bwd_ws, where the library has a kernel that uses a workspace: f32
    I/O up to 128 units runs every unit on two workgroups) on the current stream.  workspace: a device tensor of
    ttt_linear_bwd_workspace_bytes(desc) bytes, None to allocate one, False to call the entry point without.

    Counterpart of backward_multi (rust/fused/src/linear_fused_tile/backward/launch.rs:332-438).
    Returns a dict with the nine input gradients named as TttGradInputs
    (backward/launch.rs:427-437): grad_xq, grad_xk, grad_xv, grad_weight [B,H,d,d],
    grad_bias [B,H,d], grad_ttt_lr_eta, grad_token_eta [seq], grad_ln_weight, grad_ln_bias.
    """
    B, H, seq, d = xq.shape
    io = xq.dtype
    xq = _need(xq, (B, H, seq, d), io, "xq")
    xk = _need(xk, (B, H, seq, d), io, "xk")
    xv = _need(xv, (B, H, seq, d), io, "xv")
    go = _need(grad_output, (B, H, seq, d), io, "grad_output")
    lr = _need(ttt_lr_eta, (B, H, seq), io, "ttt_lr_eta")
    per_batch = weight.dim() == 4
    weight = _need(weight, (B, H, d, d) if per_batch else (H, d, d), torch.float32, "weight")
    bias = _need(bias, (B, H, d) if per_batch else (H, d), torch.float32, "bias")
    ln_weight = _need(ln_weight, (H, d), torch.float32, "ln_weight")
    ln_bias = _need(ln_bias, (H, d), torch.float32, "ln_bias")
    te = token_eta.to(torch.float32).contiguous()
    desc = TttDesc(B, H, seq, d, mini_batch, eps, checkpoint_interval, _io_dtype(xq), int(per_batch), 0,
                   int(packed_checkpoints), kernel_hint)
    check(lib().ttt_linear_bwd_supported(C.byref(desc)))
    n = lib().ttt_linear_num_checkpoints(C.byref(desc))
    w_ck = _need(weight_ckpt, (B, H, n, d, d), torch.float32, "weight_ckpt")
    b_ck = _need(bias_ckpt, (B, H, n, d), torch.float32, "bias_ckpt")
    if grad_weight_out is not None:
        grad_weight_out = _need(grad_weight_out, (B, H, d, d), torch.float32, "grad_weight_out")
        grad_bias_out = _need(grad_bias_out, (B, H, d), torch.float32, "grad_bias_out")
    dev = xq.device
    g = dict(
        grad_xq=torch.empty_like(xq), grad_xk=torch.empty_like(xq), grad_xv=torch.empty_like(xq),
        grad_weight=torch.empty((B, H, d, d), dtype=torch.float32, device=dev),
        grad_bias=torch.empty((B, H, d), dtype=torch.float32, device=dev),
        grad_ttt_lr_eta=torch.empty_like(lr),
        grad_token_eta=torch.empty((seq,), dtype=torch.float32, device=dev),
        grad_ln_weight=torch.empty((H, d), dtype=torch.float32, device=dev),
        grad_ln_bias=torch.empty((H, d), dtype=torch.float32, device=dev),
    )
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    # a desc whose backward can use a workspace (two workgroups per unit) gets one: ttt_linear_bwd_ws
    ws_bytes = lib().ttt_linear_bwd_workspace_bytes(C.byref(desc))
    if ws_bytes < 0:
        check(int(ws_bytes))
    args = (C.byref(desc), _ptr(xq), _ptr(xk), _ptr(xv), _ptr(weight), _ptr(bias), _ptr(te), _ptr(lr),
            _ptr(ln_weight), _ptr(ln_bias), _ptr(w_ck), _ptr(b_ck), _ptr(go), _ptr(grad_weight_out),
            _ptr(grad_bias_out), _ptr(g["grad_xq"]), _ptr(g["grad_xk"]), _ptr(g["grad_xv"]),
            _ptr(g["grad_weight"]), _ptr(g["grad_bias"]), _ptr(g["grad_ttt_lr_eta"]),
            _ptr(g["grad_token_eta"]), _ptr(g["grad_ln_weight"]), _ptr(g["grad_ln_bias"]))
    with torch.cuda.device(dev):
        if ws_bytes > 0 and workspace is not False:
            if workspace is None or workspace is True:
                workspace = torch.empty((int(ws_bytes),), dtype=torch.uint8, device=dev)
            if workspace.numel() * workspace.element_size() < ws_bytes:
                raise _lib.TttError(_lib.TTT_ERR_SHAPE, f"workspace holds fewer than {ws_bytes} bytes")
            check(lib().ttt_linear_bwd_ws(*args, _ptr(workspace), stream))
        else:
            check(lib().ttt_linear_bwd(*args, stream))
    return g


def ttt_mlp_forward_raw(xq, xk, xv, w1, b1, w2, b2, token_eta, ttt_lr_eta, ln_weight, ln_bias,
                        mini_batch: int, eps: float = 1e-6, kernel_hint: int = 0, save_for_backward: bool = False):
    """One call of ttt_mlp_fwd on the current stream: the fused counterpart of
    TTTMLP::forward (rust/core/src/mlp.rs:127-208 looped as rust/core/src/inner.rs:25-50).
    w1 [B,H,d,4d] or [H,d,4d], b1 [..,4d], w2 [..,4d,d], b2 [..,d].
    Returns (output, w1_out, b1_out, w2_out, b2_out), state per batch element.
    save_for_backward: call ttt_mlp_fwd_saving instead and return a sixth element, the `saved` buffer that
    ttt_mlp_backward_raw(saved=...) consumes (the backward then skips its own forward sweep)."""
    B, H, seq, d = xq.shape
    m = w1.shape[-1]
    io = xq.dtype
    xq = _need(xq, (B, H, seq, d), io, "xq")
    xk = _need(xk, (B, H, seq, d), io, "xk")
    xv = _need(xv, (B, H, seq, d), io, "xv")
    lr = _need(ttt_lr_eta, (B, H, seq), io, "ttt_lr_eta")
    per_batch = w1.dim() == 4
    lead = (B, H) if per_batch else (H,)
    if m != 4 * d:
        raise _lib.TttError(_lib.TTT_ERR_UNSUPPORTED, f"mlp_dim {m} != 4*head_dim (only expansion 4)")
    w1 = _need(w1, lead + (d, m), torch.float32, "w1")
    b1 = _need(b1, lead + (m,), torch.float32, "b1")
    w2 = _need(w2, lead + (m, d), torch.float32, "w2")
    b2 = _need(b2, lead + (d,), torch.float32, "b2")
    ln_weight = _need(ln_weight, (H, d), torch.float32, "ln_weight")
    ln_bias = _need(ln_bias, (H, d), torch.float32, "ln_bias")
    if token_eta.numel() < mini_batch:
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, "token_eta shorter than mini_batch")
    te = token_eta.to(torch.float32).contiguous()
    desc = TttDesc(B, H, seq, d, mini_batch, eps, 1, _io_dtype(xq), int(per_batch), 0, 0, kernel_hint)
    check(lib().ttt_mlp_supported(C.byref(desc)))
    dev = xq.device
    f32 = dict(dtype=torch.float32, device=dev)
    out = torch.empty_like(xq)
    o = [torch.empty((B, H, d, m), **f32), torch.empty((B, H, m), **f32),
         torch.empty((B, H, m, d), **f32), torch.empty((B, H, d), **f32)]
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    with torch.cuda.device(dev):
        if save_for_backward:
            check(lib().ttt_mlp_fwd_saving_supported(C.byref(desc)))
            saved = torch.empty((lib().ttt_mlp_bwd_workspace_bytes(C.byref(desc)) + 3) // 4, **f32)
            check(lib().ttt_mlp_fwd_saving(C.byref(desc), _ptr(xq), _ptr(xk), _ptr(xv), _ptr(w1), _ptr(b1), _ptr(w2),
                                           _ptr(b2), _ptr(te), _ptr(lr), _ptr(ln_weight), _ptr(ln_bias), _ptr(out),
                                           *[_ptr(x) for x in o], _ptr(saved), stream))
            return (out, *o, saved)
        check(lib().ttt_mlp_fwd(C.byref(desc), _ptr(xq), _ptr(xk), _ptr(xv), _ptr(w1), _ptr(b1), _ptr(w2),
                                _ptr(b2), _ptr(te), _ptr(lr), _ptr(ln_weight), _ptr(ln_bias), _ptr(out),
                                *[_ptr(x) for x in o], stream))
    return (out, *o)


def ttt_mlpn_forward_raw(xq, xk, xv, weights, biases, token_eta, ttt_lr_eta, ln_weight, ln_bias, mini_batch: int,
                         eps: float = 1e-6):
    """One call of ttt_mlpn_fwd on the current stream: TTTMLP2/3/4::forward (rust/core/src/mlp2.rs, mlp3.rs, mlp4.rs
    looped as rust/core/src/inner.rs:25-50).  weights / biases: lists of the n_hidden + 1 layers, [H,in,out] / [H,out] or
    with a leading batch dimension.  Returns (output, weights_out, biases_out), state per batch element."""
    B, H, seq, d = xq.shape
    io = xq.dtype
    n_hidden = len(weights) - 1
    m = 4 * d
    dims = [d] + [m] * n_hidden + [d]
    xq = _need(xq, (B, H, seq, d), io, "xq")
    xk = _need(xk, (B, H, seq, d), io, "xk")
    xv = _need(xv, (B, H, seq, d), io, "xv")
    per_batch = weights[0].dim() == 4
    lead = (B, H) if per_batch else (H,)
    Ws = [_need(w, lead + (dims[i], dims[i + 1]), torch.float32, f"weights[{i}]") for i, w in enumerate(weights)]
    bs = [_need(b, lead + (dims[i + 1],), torch.float32, f"biases[{i}]") for i, b in enumerate(biases)]
    te = _need(token_eta[:mini_batch], (mini_batch,), torch.float32, "token_eta")
    lr = _need(ttt_lr_eta, (B, H, seq), io, "ttt_lr_eta")
    gam = _need(ln_weight, (H, d), torch.float32, "ln_weight")
    bet = _need(ln_bias, (H, d), torch.float32, "ln_bias")
    dev = xq.device
    desc = TttDesc(B, H, seq, d, mini_batch, eps, 1, _io_dtype(xq), 1 if per_batch else 0, 0, 0, 0)
    check(lib().ttt_mlpn_supported(C.byref(desc), n_hidden))
    out = torch.empty((B, H, seq, d), dtype=io, device=dev)
    Wo = [torch.empty((B, H, dims[i], dims[i + 1]), dtype=torch.float32, device=dev) for i in range(n_hidden + 1)]
    bo = [torch.empty((B, H, dims[i + 1]), dtype=torch.float32, device=dev) for i in range(n_hidden + 1)]
    arr = lambda ts: (C.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    with torch.cuda.device(dev):
        check(lib().ttt_mlpn_fwd(C.byref(desc), n_hidden, _ptr(xq), _ptr(xk), _ptr(xv), arr(Ws), arr(bs), _ptr(te),
                                 _ptr(lr), _ptr(gam), _ptr(bet), _ptr(out), arr(Wo), arr(bo), stream))
    return out, Wo, bo


def ttt_mlp_backward_raw(xq, xk, xv, w1, b1, w2, b2, token_eta, ttt_lr_eta, ln_weight, ln_bias, d_out,
                         mini_batch: int, eps: float = 1e-6, d_state_out=None, static_scratch: bool = False,
                         into=None, kernel_hint: int = 0, saved=None):
    """One call of ttt_mlp_bwd on the current stream: gradients of the TTT-MLP inner loop
    (rust/core/src/mlp.rs:127-208 looped as rust/core/src/inner.rs:25-50; the reference gets them
    from Burn autodiff).  Arguments as ttt_mlp_forward_raw plus d_out [B,H,seq,d] and the optional
    upstream gradients of the final state d_state_out = (dW1, db1, dW2, db2), per batch element.
    Returns a dict: d_xq, d_xk, d_xv, d_W1 [B,H,d,4d], d_b1, d_W2, d_b2 (per batch element), d_lr,
    d_token_eta [seq], d_gamma, d_beta [H,d].
    static_scratch: call ttt_mlp_bwd_static (the library's built-in scratch buffer instead of a workspace
    allocated here); `into`: a dict returned by an earlier call of the same shape, whose tensors receive the
    gradients (with both, the call allocates no device memory).  kernel_hint: TTT_HINT_F32_PRODUCTS keeps the
    reverse scan's products in f32 where it would round their operands to bf16 (bf16 I/O, head_dim <= 96).
    saved: the buffer a forward with save_for_backward=True returned (same inputs, same hint): ttt_mlp_bwd_saved, which
    consumes it."""
    B, H, seq, d = xq.shape
    m = w1.shape[-1]
    io = xq.dtype
    xq = _need(xq, (B, H, seq, d), io, "xq")
    xk = _need(xk, (B, H, seq, d), io, "xk")
    xv = _need(xv, (B, H, seq, d), io, "xv")
    d_out = _need(d_out, (B, H, seq, d), io, "d_out")
    lr = _need(ttt_lr_eta, (B, H, seq), io, "ttt_lr_eta")
    per_batch = w1.dim() == 4
    lead = (B, H) if per_batch else (H,)
    if m != 4 * d:
        raise _lib.TttError(_lib.TTT_ERR_UNSUPPORTED, f"mlp_dim {m} != 4*head_dim (only expansion 4)")
    w1 = _need(w1, lead + (d, m), torch.float32, "w1")
    b1 = _need(b1, lead + (m,), torch.float32, "b1")
    w2 = _need(w2, lead + (m, d), torch.float32, "w2")
    b2 = _need(b2, lead + (d,), torch.float32, "b2")
    ln_weight = _need(ln_weight, (H, d), torch.float32, "ln_weight")
    ln_bias = _need(ln_bias, (H, d), torch.float32, "ln_bias")
    if token_eta.numel() < mini_batch:
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, "token_eta shorter than mini_batch")
    te = token_eta.to(torch.float32).contiguous()
    desc = TttDesc(B, H, seq, d, mini_batch, eps, 1, _io_dtype(xq), int(per_batch), 0)
    desc.kernel_hint = int(kernel_hint)
    check(lib().ttt_mlp_supported(C.byref(desc)))
    dev = xq.device
    f32 = dict(dtype=torch.float32, device=dev)
    shapes = [(B, H, d, m), (B, H, m), (B, H, m, d), (B, H, d)]
    up = [None] * 4
    if d_state_out is not None:
        up = [_need(g, sh, torch.float32, "d_state_out") for g, sh in zip(d_state_out, shapes)]
    if into is not None:
        g_act = [into["d_xq"], into["d_xk"], into["d_xv"]]
        g_st = [into["d_W1"], into["d_b1"], into["d_W2"], into["d_b2"]]
        g_lr, g_te, g_gam, g_bet = into["d_lr"], into["d_token_eta"], into["d_gamma"], into["d_beta"]
        for t, sh in zip(g_act + g_st + [g_lr, g_te, g_gam, g_bet],
                         [xq.shape] * 3 + shapes + [lr.shape, (seq,), (H, d), (H, d)]):
            if tuple(t.shape) != tuple(sh) or not t.is_contiguous() or not t.is_cuda:
                raise _lib.TttError(_lib.TTT_ERR_SHAPE, "into: a gradient tensor has the wrong shape or layout")
    else:
        g_act = [torch.empty_like(xq) for _ in range(3)]
        g_st = [torch.empty(sh, **f32) for sh in shapes]
        g_lr = torch.empty_like(lr)
        g_te = torch.empty(seq, **f32)
        g_gam, g_bet = torch.empty((H, d), **f32), torch.empty((H, d), **f32)
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    null = C.c_void_p(None)
    args = [C.byref(desc), _ptr(xq), _ptr(xk), _ptr(xv), _ptr(w1), _ptr(b1), _ptr(w2), _ptr(b2), _ptr(te), _ptr(lr),
            _ptr(ln_weight), _ptr(ln_bias), _ptr(d_out), *[null if g is None else _ptr(g) for g in up],
            *[_ptr(g) for g in g_act], *[_ptr(g) for g in g_st], _ptr(g_lr), _ptr(g_te), _ptr(g_gam), _ptr(g_bet)]
    with torch.cuda.device(dev):
        if saved is not None:
            if saved.numel() * saved.element_size() < lib().ttt_mlp_bwd_workspace_bytes(C.byref(desc)):
                raise _lib.TttError(_lib.TTT_ERR_SHAPE, "saved is smaller than this desc's workspace (a forward with "
                                                         "another kernel_hint?)")
            check(lib().ttt_mlp_bwd_saved(*args, _ptr(saved), stream))
        elif static_scratch:
            check(lib().ttt_mlp_bwd_static(*args, stream))
        else:
            nbytes = lib().ttt_mlp_bwd_workspace_bytes(C.byref(desc))
            if nbytes < 0:
                raise _lib.TttError(_lib.TTT_ERR_SHAPE, "ttt_mlp_bwd_workspace_bytes failed")
            ws = torch.empty((nbytes + 3) // 4, **f32)
            check(lib().ttt_mlp_bwd(*args, _ptr(ws), stream))
    return dict(d_xq=g_act[0], d_xk=g_act[1], d_xv=g_act[2], d_W1=g_st[0], d_b1=g_st[1], d_W2=g_st[2],
                d_b2=g_st[3], d_lr=g_lr, d_token_eta=g_te, d_gamma=g_gam, d_beta=g_bet)


@dataclass
class TTTMLPState:
    """mlp.rs:43-53: w1 [B,H,d,4d], b1 [B,H,4d], w2 [B,H,4d,d], b2 [B,H,d], always f32."""
    w1: torch.Tensor
    b1: torch.Tensor
    w2: torch.Tensor
    b2: torch.Tensor


class FusedMlp:
    """Fused TTT-MLP layer with the TTTMLP parameter set (mlp.rs:29-41) and the TTTInnerModel
    surface (inner.rs:13-58)."""

    def __init__(self, config: ModelConfig, w1_init, b1_init, w2_init, b2_init, ln_weight, ln_bias):
        H, d = config.num_heads, config.head_dim
        m = config.ttt.mlp_expansion_factor * d
        self.config = config
        self.w1_init = _need(w1_init, (H, d, m), torch.float32, "w1_init")
        self.b1_init = _need(b1_init, (H, m), torch.float32, "b1_init")
        self.w2_init = _need(w2_init, (H, m, d), torch.float32, "w2_init")
        self.b2_init = _need(b2_init, (H, d), torch.float32, "b2_init")
        self.ln_weight = _need(ln_weight, (H, d), torch.float32, "ln_weight")
        self.ln_bias = _need(ln_bias, (H, d), torch.float32, "ln_bias")

    @staticmethod
    def name() -> str:
        return "FusedTTTMLP"

    @classmethod
    def new(cls, config: ModelConfig, device, generator: Optional[torch.Generator] = None):
        """TTTMLP::new (mlp.rs:76-113): every parameter ~ Normal(0, 0.02)."""
        H, d = config.num_heads, config.head_dim
        m = config.ttt.mlp_expansion_factor * d

        def init(*shape):
            return (torch.randn(*shape, generator=generator, dtype=torch.float32) * 0.02).to(device)

        return cls(config, init(H, d, m), init(H, m), init(H, m, d), init(H, d), init(H, d), init(H, d))

    def get_config(self) -> ModelConfig:
        return self.config

    def init_state(self, batch_size: int) -> TTTMLPState:
        """mlp.rs:119-125."""
        rep = lambda p: p.unsqueeze(0).repeat(batch_size, *([1] * p.dim()))
        return TTTMLPState(rep(self.w1_init), rep(self.b1_init), rep(self.w2_init), rep(self.b2_init))

    def _launch(self, state: TTTMLPState, inputs: TTTInputsInner, mini_batch: int):
        out, state.w1, state.b1, state.w2, state.b2 = ttt_mlp_forward_raw(
            inputs.qkv.xq, inputs.qkv.xk, inputs.qkv.xv, state.w1, state.b1, state.w2, state.b2,
            inputs.token_eta, inputs.ttt_lr_eta, self.ln_weight, self.ln_bias, mini_batch,
            self.config.ttt.epsilon)
        return out

    def forward(self, state: TTTMLPState, inputs: TTTInputsInner) -> torch.Tensor:
        """inner.rs:25-50 in at most two launches: all full mini-batches, then the remainder."""
        K = self.config.ttt.mini_batch_size
        seq = inputs.qkv.xq.shape[2]
        full = (seq // K) * K
        outs = []
        if full > 0:
            outs.append(self._launch(state, inputs.slice_seq(range(0, full)), K))
        if full < seq:
            outs.append(self._launch(state, inputs.slice_seq(range(full, seq)), seq - full))
        return outs[0] if len(outs) == 1 else torch.cat(outs, 2)

    def forward_mini_batch(self, state: TTTMLPState, inputs: TTTInputsInner, r: range) -> torch.Tensor:
        if len(r) > self.config.ttt.mini_batch_size or len(r) == 0:
            raise _lib.TttError(_lib.TTT_ERR_SHAPE, "range longer than mini_batch_size")
        return self._launch(state, inputs.slice_seq(r), len(r))

    def backward(self, state0: Optional[TTTMLPState], inputs: TTTInputsInner, grad_output, grad_state_out=None):
        """Gradients of forward() over a sequence that is a multiple of mini_batch_size, starting from
        state0 (None: the [H,..] parameters broadcast over batch, init_state).  The reference gets these
        from Burn autodiff over mlp.rs:127-208.  Returns the dict of ttt_mlp_backward_raw."""
        st = (self.w1_init, self.b1_init, self.w2_init, self.b2_init) if state0 is None else \
            (state0.w1, state0.b1, state0.w2, state0.b2)
        return ttt_mlp_backward_raw(inputs.qkv.xq, inputs.qkv.xk, inputs.qkv.xv, *st, inputs.token_eta,
                                    inputs.ttt_lr_eta, self.ln_weight, self.ln_bias, grad_output,
                                    self.config.ttt.mini_batch_size, self.config.ttt.epsilon,
                                    d_state_out=grad_state_out)


class FusedTileMulti:
    """`fused-tile-multi` TTT-Linear layer: Fused<B, TTTLinear<B>, TileMultiKernel>.

    Holds the same parameters as TTTLinear (weight_init [H,d,d], bias_init [H,d], LayerNorm
    weight/bias [H,d]; linear.rs:17-25) so records are interchangeable with the plain layer
    (rust/fused/src/lib.rs:183-277).
    """

    def __init__(self, config: ModelConfig, weight_init, bias_init, ln_weight, ln_bias):
        H, d = config.num_heads, config.head_dim
        self.config = config
        self.weight_init = _need(weight_init, (H, d, d), torch.float32, "weight_init")
        self.bias_init = _need(bias_init, (H, d), torch.float32, "bias_init")
        self.ln_weight = _need(ln_weight, (H, d), torch.float32, "ln_weight")
        self.ln_bias = _need(ln_bias, (H, d), torch.float32, "ln_bias")

    @staticmethod
    def name() -> str:
        return "FusedTileMultiTTTLinear"  # wrapper.rs:85-87

    @classmethod
    def new(cls, config: ModelConfig, device, generator: Optional[torch.Generator] = None):
        """TTTLinear::new (linear.rs:54-78): every parameter ~ Normal(0, 0.02)."""
        H, d = config.num_heads, config.head_dim

        def init(*shape):
            return (torch.randn(*shape, generator=generator, dtype=torch.float32) * 0.02).to(device)

        return cls(config, init(H, d, d), init(H, d), init(H, d), init(H, d))

    def get_config(self) -> ModelConfig:
        return self.config

    def init_state(self, batch_size: int) -> TTTLinearState:
        """linear.rs:84-89: parameters repeated over the batch."""
        return TTTLinearState(self.weight_init.unsqueeze(0).repeat(batch_size, 1, 1, 1),
                              self.bias_init.unsqueeze(0).repeat(batch_size, 1, 1))

    def _launch(self, state: TTTLinearState, inputs: TTTInputsInner, mini_batch: int, out=None):
        t = self.config.ttt
        out, w, b = ttt_linear_forward_raw(
            inputs.qkv.xq, inputs.qkv.xk, inputs.qkv.xv, state.weight, state.bias, inputs.token_eta,
            inputs.ttt_lr_eta, self.ln_weight, self.ln_bias, mini_batch, t.epsilon,
            t.checkpoint_interval, out=out)
        state.weight, state.bias = w, b
        return out

    def forward(self, state: TTTLinearState, inputs: TTTInputsInner) -> torch.Tensor:
        """wrapper.rs:102-164: all full mini-batches in one launch; a trailing remainder is one
        short mini-batch, as the Burn-op model does it (inner.rs:40-47)."""
        K = self.config.ttt.mini_batch_size
        seq = inputs.qkv.xq.shape[2]
        full = (seq // K) * K
        # one output tensor; both launches read and write sequence windows in place
        output = torch.empty(inputs.qkv.xq.shape, dtype=inputs.qkv.xq.dtype, device=inputs.qkv.xq.device)
        if full > 0:
            self._launch(state, inputs.slice_seq(range(0, full)), K, out=output[:, :, :full])
        if full < seq:
            self._launch(state, inputs.slice_seq(range(full, seq)), seq - full, out=output[:, :, full:])
        return output

    def forward_mini_batch(self, state: TTTLinearState, inputs: TTTInputsInner, r: range) -> torch.Tensor:
        """wrapper.rs:166-211: one mini-batch (len(r) <= mini_batch_size)."""
        if len(r) > self.config.ttt.mini_batch_size or len(r) == 0:
            raise _lib.TttError(_lib.TTT_ERR_SHAPE, "range longer than mini_batch_size")
        return self._launch(state, inputs.slice_seq(r), len(r))


@dataclass
class TTTLinearAdamState:
    """linear_adam.rs:28-44: state, first and second moments (per batch element, f32) and the step counter."""
    weight: torch.Tensor
    bias: torch.Tensor
    weight_m: torch.Tensor
    bias_m: torch.Tensor
    weight_v: torch.Tensor
    bias_v: torch.Tensor
    step: int = 0


@dataclass
class TTTLinearAdamConfig:
    """linear_adam.rs:46-62."""
    beta1: float = 0.9
    beta2: float = 0.999
    epsilon: float = 1e-8
    lr: float = 1e-3


class FusedLinearAdam:
    """TTTLinearAdam (rust/core/src/linear_adam.rs) on the fused kernel: the parameters of TTTLinear, an Adam step
    on the eta-weighted gradients per mini-batch instead of the plain update."""

    def __init__(self, config: ModelConfig, adam: TTTLinearAdamConfig, weight_init, bias_init, ln_weight, ln_bias):
        H, d = config.num_heads, config.head_dim
        self.config, self.adam = config, adam
        self.weight_init = _need(weight_init, (H, d, d), torch.float32, "weight_init")
        self.bias_init = _need(bias_init, (H, d), torch.float32, "bias_init")
        self.ln_weight = _need(ln_weight, (H, d), torch.float32, "ln_weight")
        self.ln_bias = _need(ln_bias, (H, d), torch.float32, "ln_bias")

    @staticmethod
    def name() -> str:
        return "TTTLinearAdam"  # linear_adam.rs:134-136

    def get_config(self) -> ModelConfig:
        return self.config

    def init_state(self, batch_size: int) -> TTTLinearAdamState:
        """linear_adam.rs:164-177: parameters repeated over the batch, zero moments, step 0."""
        w = self.weight_init.unsqueeze(0).repeat(batch_size, 1, 1, 1)
        b = self.bias_init.unsqueeze(0).repeat(batch_size, 1, 1)
        return TTTLinearAdamState(w, b, torch.zeros_like(w), torch.zeros_like(b), torch.zeros_like(w),
                                  torch.zeros_like(b), 0)

    def _launch(self, state: TTTLinearAdamState, inputs: TTTInputsInner, mini_batch: int):
        a = self.adam
        out, w, b, mo, step = ttt_linear_adam_forward_raw(
            inputs.qkv.xq, inputs.qkv.xk, inputs.qkv.xv, state.weight, state.bias, inputs.token_eta,
            inputs.ttt_lr_eta, self.ln_weight, self.ln_bias, mini_batch, a.beta1, a.beta2, a.epsilon, a.lr,
            moments=(state.weight_m, state.bias_m, state.weight_v, state.bias_v), step=state.step,
            eps=self.config.ttt.epsilon)
        state.weight, state.bias = w, b
        state.weight_m, state.bias_m, state.weight_v, state.bias_v = mo
        state.step = step
        return out

    def forward(self, state: TTTLinearAdamState, inputs: TTTInputsInner) -> torch.Tensor:
        """inner.rs:25-50: all full mini-batches in one launch, a trailing remainder as one short mini-batch."""
        K = self.config.ttt.mini_batch_size
        seq = inputs.qkv.xq.shape[2]
        full = (seq // K) * K
        outs = []
        if full > 0:
            outs.append(self._launch(state, inputs.slice_seq(range(0, full)), K))
        if full < seq:
            outs.append(self._launch(state, inputs.slice_seq(range(full, seq)), seq - full))
        return outs[0] if len(outs) == 1 else torch.cat(outs, 2)

    def forward_mini_batch(self, state: TTTLinearAdamState, inputs: TTTInputsInner, r: range) -> torch.Tensor:
        if len(r) > self.config.ttt.mini_batch_size or len(r) == 0:
            raise _lib.TttError(_lib.TTT_ERR_SHAPE, "range longer than mini_batch_size")
        return self._launch(state, inputs.slice_seq(r), len(r))


@dataclass
class TTTMLPNState:
    """mlp2.rs:38-53, mlp3.rs:42-53, mlp4.rs:46-59: the n_hidden + 1 weight layers [B,H,in,out] and biases [B,H,out],
    always f32."""
    weights: list
    biases: list


class FusedMlpN:
    """TTTMLP2 / TTTMLP3 / TTTMLP4 (rust/core/src/mlp2.rs, mlp3.rs, mlp4.rs) on the fused kernel: d -> 4d -> ... -> 4d
    -> d with 2, 3 or 4 hidden layers, the TTTInnerModel interface of rust/core/src/inner.rs:13-58."""

    def __init__(self, config: ModelConfig, weights_init, biases_init, ln_weight, ln_bias):
        H, d = config.num_heads, config.head_dim
        n = len(weights_init) - 1
        if n < 2 or n > 4 or len(biases_init) != n + 1:
            raise _lib.TttError(_lib.TTT_ERR_UNSUPPORTED, "FusedMlpN: 2, 3 or 4 hidden layers")
        dims = [d] + [4 * d] * n + [d]
        self.config, self.n_hidden = config, n
        self.weights_init = [_need(w, (H, dims[i], dims[i + 1]), torch.float32, f"weights_init[{i}]")
                             for i, w in enumerate(weights_init)]
        self.biases_init = [_need(b, (H, dims[i + 1]), torch.float32, f"biases_init[{i}]")
                            for i, b in enumerate(biases_init)]
        self.ln_weight = _need(ln_weight, (H, d), torch.float32, "ln_weight")
        self.ln_bias = _need(ln_bias, (H, d), torch.float32, "ln_bias")

    def name(self) -> str:
        return f"TTTMLP{self.n_hidden}"  # mlp2.rs:70-72, mlp3.rs:70-72, mlp4.rs:76-78

    def get_config(self) -> ModelConfig:
        return self.config

    def init_state(self, batch_size: int) -> TTTMLPNState:
        """mlp2.rs:129-145 and its siblings: the parameters repeated over the batch."""
        rep = lambda t: t.unsqueeze(0).repeat(batch_size, *([1] * t.dim()))
        return TTTMLPNState([rep(w) for w in self.weights_init], [rep(b) for b in self.biases_init])

    def _launch(self, state: TTTMLPNState, inputs: TTTInputsInner, mini_batch: int):
        out, ws, bs = ttt_mlpn_forward_raw(inputs.qkv.xq, inputs.qkv.xk, inputs.qkv.xv, state.weights, state.biases,
                                           inputs.token_eta, inputs.ttt_lr_eta, self.ln_weight, self.ln_bias,
                                           mini_batch, self.config.ttt.epsilon)
        state.weights, state.biases = ws, bs
        return out

    def forward(self, state: TTTMLPNState, inputs: TTTInputsInner) -> torch.Tensor:
        """inner.rs:25-50: all full mini-batches in one launch, a trailing remainder as one short mini-batch."""
        K = self.config.ttt.mini_batch_size
        seq = inputs.qkv.xq.shape[2]
        full = (seq // K) * K
        outs = []
        if full > 0:
            outs.append(self._launch(state, inputs.slice_seq(range(0, full)), K))
        if full < seq:
            outs.append(self._launch(state, inputs.slice_seq(range(full, seq)), seq - full))
        return outs[0] if len(outs) == 1 else torch.cat(outs, 2)

    def forward_mini_batch(self, state: TTTMLPNState, inputs: TTTInputsInner, r: range) -> torch.Tensor:
        if len(r) > self.config.ttt.mini_batch_size or len(r) == 0:
            raise _lib.TttError(_lib.TTT_ERR_SHAPE, "range longer than mini_batch_size")
        return self._launch(state, inputs.slice_seq(r), len(r))


def ttt_stack_workspace_bytes(B: int, H: int, seq: int, d: int, mini_batch: int, io: torch.dtype, mlp_flags,
                              chunk_tokens: int = 0) -> int:
    """ttt_stack_fwd_workspace_bytes for a stack whose layer l is TTT-MLP where mlp_flags[l] is true."""
    desc = TttDesc(B, H, seq, d, mini_batch, 1e-6, 1, _lib.TTT_BF16 if io == torch.bfloat16 else _lib.TTT_F32)
    arr = (_lib.TttStackLayer * len(mlp_flags))()
    for a, f in zip(arr, mlp_flags):
        a.kind = 1 if f else 0
    n = lib().ttt_stack_fwd_workspace_bytes(C.byref(desc), len(mlp_flags), arr, chunk_tokens)
    if n < 0:
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, lib().ttt_last_error().decode())
    return n


def mlp_fwd_lost_workgroups() -> int:
    """ttt_mlp_fwd_lost_workgroups of the current device: how many workgroups of the two-CU TTT-MLP forward
    (head_dim 128, bf16 I/O) gave up waiting for their partner since the library was loaded.  A blocking copy from
    the device; meaningful once the work in question has finished."""
    n = C.c_int64(0)
    check(lib().ttt_mlp_fwd_lost_workgroups(C.byref(n)))
    return n.value


def ttt_stack_forward_raw(layers, token_eta, mini_batch: int, eps: float = 1e-6, kernel_hint: int = 0,
                          workspace: Optional[torch.Tensor] = None, chunk_tokens: int = 0,
                          aux_stream: Optional[torch.cuda.Stream] = None, check_lost: Optional[bool] = None):
    """One call of ttt_stack_fwd on the current stream: inner models applied layer by layer, layer l on
    xq = x + pq, xk = x + pk, xv = x + pv with x the previous layer's output (0 for the first layer).
    chunk_tokens > 0 runs the layers as a wavefront over sequence windows of that many tokens (layer l + 1 works on
    a window as soon as layer l has left it; windows that are ready together share a launch); aux_stream, a second
    torch.cuda.Stream, lets the TTT-MLP launches run beside the TTT-Linear ones.
    layers: list of dicts with pq, pk, pv [B,H,seq,d], lr [B,H,seq], gamma, beta [H,d] and either W0, b0
    (TTT-Linear) or W1, b1, W2, b2 (TTT-MLP), parameters [H,..].  Returns (out, states) with states[l] the final
    state tensors of layer l (per batch element).
    check_lost: a stack with a TTT-MLP layer at head_dim 128 and bf16 I/O runs the two-CU kernel, whose failure
    (a workgroup that waited for its partner in vain) shows only in the data (NaN) and in the device's status word.
    With check_lost the call waits for the device, reads that word before and after and raises if it moved.
    Default (None): checked unless the current stream is being captured into a graph; callers that must not
    synchronise (timed loops) pass False and compare mlp_fwd_lost_workgroups() around their own region."""
    B, H, seq, d = layers[0]["pq"].shape
    io = layers[0]["pq"].dtype
    dev = layers[0]["pq"].device
    f32 = dict(dtype=torch.float32, device=dev)
    desc = TttDesc(B, H, seq, d, mini_batch, eps, 1, _io_dtype(layers[0]["pq"]), 0, 0, 0, kernel_hint)
    te = _need(token_eta.to(torch.float32), (token_eta.numel(),), torch.float32, "token_eta")
    if te.numel() < mini_batch:
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, "token_eta shorter than mini_batch")
    arr = (_lib.TttStackLayer * len(layers))()
    keep, states = [], []
    for i, L in enumerate(layers):
        mlp = "W2" in L
        m = 4 * d
        t = {k: _need(L[k], (B, H, seq, d), io, k) for k in ("pq", "pk", "pv")}
        t["lr"] = _need(L["lr"], (B, H, seq), io, "lr")
        t["gamma"] = _need(L["gamma"], (H, d), torch.float32, "gamma")
        t["beta"] = _need(L["beta"], (H, d), torch.float32, "beta")
        if mlp:
            t["W1"] = _need(L["W1"], (H, d, m), torch.float32, "W1")
            t["b1"] = _need(L["b1"], (H, m), torch.float32, "b1")
            t["W2"] = _need(L["W2"], (H, m, d), torch.float32, "W2")
            t["b2"] = _need(L["b2"], (H, d), torch.float32, "b2")
            st = [torch.empty((B, H, d, m), **f32), torch.empty((B, H, m), **f32), torch.empty((B, H, m, d), **f32),
                  torch.empty((B, H, d), **f32)]
        else:
            t["W1"] = _need(L["W0"], (H, d, d), torch.float32, "W0")
            t["b1"] = _need(L["b0"], (H, d), torch.float32, "b0")
            st = [torch.empty((B, H, d, d), **f32), torch.empty((B, H, d), **f32)]
        keep.append(t)
        states.append(st)
        a = arr[i]
        a.kind = 1 if mlp else 0
        for k in ("pq", "pk", "pv", "W1", "b1", "lr", "gamma", "beta"):
            setattr(a, k, t[k].data_ptr())
        a.W2 = t["W2"].data_ptr() if mlp else None
        a.b2 = t["b2"].data_ptr() if mlp else None
        a.W1_out, a.b1_out = st[0].data_ptr(), st[1].data_ptr()
        a.W2_out = st[2].data_ptr() if mlp else None
        a.b2_out = st[3].data_ptr() if mlp else None
    nbytes = lib().ttt_stack_fwd_workspace_bytes(C.byref(desc), len(layers), arr, chunk_tokens)
    if nbytes < 0:
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, lib().ttt_last_error().decode())
    if workspace is None:
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    elif workspace.numel() * workspace.element_size() < nbytes:
        raise _lib.TttError(_lib.TTT_ERR_SHAPE, "workspace too small")
    out = torch.empty((B, H, seq, d), dtype=io, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    two_cu = (d == 128 or (d == 96 and kernel_hint & _lib.TTT_HINT_TWO_CU)) and io == torch.bfloat16 and \
        any("W2" in L for L in layers) and not (kernel_hint & _lib.TTT_HINT_LDS_TILES)
    if check_lost is None:
        check_lost = two_cu and not torch.cuda.is_current_stream_capturing()
    with torch.cuda.device(dev):
        lost_before = 0
        if check_lost and two_cu:
            torch.cuda.synchronize(dev)
            lost_before = mlp_fwd_lost_workgroups()
        check(lib().ttt_stack_fwd(C.byref(desc), len(layers), arr, _ptr(te), _ptr(out), _ptr(workspace),
                                  chunk_tokens, C.c_void_p(aux_stream.cuda_stream) if aux_stream is not None else None,
                                  stream))
        if check_lost and two_cu:
            torch.cuda.synchronize(dev)
            lost = mlp_fwd_lost_workgroups() - lost_before
            if lost and not (kernel_hint & _lib.TTT_HINT_TEST_LOST_PARTNER):
                raise _lib.TttError(_lib.TTT_ERR_HIP, f"ttt_stack_fwd: {lost} workgroups of the two-CU TTT-MLP kernel "
                                    "waited for their partner in vain; the outputs of their units are NaN")
    # aux_stream reads and writes tensors that torch's allocator ties to the current stream only; the call joins
    # it into the current stream before it returns, so later work on that stream is ordered after it
    return out, states


# --------------------------------------------------------------------------- either side of the inner loop
def rope_cos_sin(seq_len: int, offset: int, wrap: Optional[int], head_dim: int, device, base: float = 10000.0):
    """RotaryEmbeddingConfig::init + RotaryEmbedding::get_cos_sin (rust/core/src/util.rs:266-322) in f32:
    returns (cos, sin) [seq_len, head_dim/2] (the reference repeats this half twice)."""
    half = head_dim // 2
    inv_freq = torch.tensor([1.0 / base ** ((2 * i) / head_dim) for i in range(half)], dtype=torch.float32)
    pos = torch.arange(seq_len, dtype=torch.float32) + float(offset)
    if wrap is not None:
        pos = torch.remainder(pos, float(wrap))
    freqs = pos[:, None] * inv_freq[None, :]
    return freqs.cos().to(device), freqs.sin().to(device)


def ttt_lr_eta_logit_grad(grad_ttt_lr_eta, lr_logits, base_lr: float, head_dim: int):
    """Gradient w.r.t. the lr-gate logits from grad_ttt_lr_eta (an output of ttt_linear_backward_raw /
    ttt_mlp_backward_raw): the chain through ttt_lr_eta = base_lr * sigmoid(logit) / head_dim (get_lr,
    rust/layer/src/ttt.rs:205-227).  The reference leaves this step to Burn autodiff outside the fused kernel's
    boundary; here it is one elementwise expression on the caller's device, in f32."""
    s = torch.sigmoid(lr_logits.float())
    return grad_ttt_lr_eta.float() * (base_lr / head_dim) * s * (1.0 - s)


def inner_loop_inputs_raw(xq, xk, xv, lr_logits, lr_bias, base_lr: float, token_idx, learnable_token_idx,
                          mini_batch: int, rope=None, pos_offset: int = 0, pos_wrap: int = 0) -> TTTInputsInner:
    """One call of ttt_inner_inputs: TTT::get_inner_loop_inputs after the projections
    (rust/layer/src/ttt.rs:147-194, 205-227, 247-268).  xq,xk,xv [B,seq,H,d]; lr_logits [B,seq,H];
    rope = (cos, sin) tables [npos, d/2] f32 or None."""
    B, seq, H, d = xq.shape
    io = xq.dtype
    xq = _need(xq, (B, seq, H, d), io, "xq")
    xk = _need(xk, (B, seq, H, d), io, "xk")
    xv = _need(xv, (B, seq, H, d), io, "xv")
    lg = _need(lr_logits, (B, seq, H), io, "lr_logits")
    lb = _need(lr_bias.reshape(-1), (H,), torch.float32, "lr_bias")
    ti = _need(token_idx, (mini_batch,), torch.float32, "token_idx")
    lti = _need(learnable_token_idx, (mini_batch,), torch.float32, "learnable_token_idx")
    null = C.c_void_p(None)
    cos = sin = None
    if rope is not None:
        cos = _need(rope[0], (rope[0].shape[0], d // 2), torch.float32, "rope cos")
        sin = _need(rope[1], (rope[0].shape[0], d // 2), torch.float32, "rope sin")
        last = (pos_offset + seq - 1) if pos_wrap == 0 else min(pos_wrap - 1, pos_offset + seq - 1)
        if last >= cos.shape[0]:
            raise _lib.TttError(_lib.TTT_ERR_SHAPE, "rope table shorter than the positions used")
    dev = xq.device
    q, k, v = (torch.empty((B, H, seq, d), dtype=io, device=dev) for _ in range(3))
    lr = torch.empty((B, H, seq), dtype=io, device=dev)
    te = torch.empty(seq, dtype=torch.float32, device=dev)
    desc = TttDesc(B, H, seq, d, mini_batch, 0.0, 1, _io_dtype(xq), 0, 0)
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    with torch.cuda.device(dev):
        check(lib().ttt_inner_inputs(C.byref(desc), _ptr(xq), _ptr(xk), _ptr(xv), _ptr(lg), _ptr(lb),
                                     C.c_float(base_lr), _ptr(ti), _ptr(lti),
                                     null if cos is None else _ptr(cos), null if sin is None else _ptr(sin),
                                     pos_offset, pos_wrap, _ptr(q), _ptr(k), _ptr(v), _ptr(lr), _ptr(te), stream))
    return TTTInputsInner(Qkv(q, k, v), te, lr)


def ttt_linear_forward_fused_inputs_raw(xq, xk, xv, lr_logits, lr_bias, base_lr: float, token_idx,
                                        learnable_token_idx, weight, bias, ln_weight, ln_bias, mini_batch: int,
                                        rope=None, pos_offset: int = 0, pos_wrap: int = 0, eps: float = 1e-6,
                                        checkpoint_interval: int = 1, want_checkpoints: bool = False,
                                        packed_checkpoints: int = 0, save_inputs: bool = False):
    """One call of ttt_linear_fwd_fused_inputs: inner_loop_inputs_raw and ttt_linear_forward_raw in one kernel
    (rust/layer/src/ttt.rs:147-268 followed by rust/kernels/src/kernel.rs:62-69).  xq,xk,xv [B,seq,H,d];
    lr_logits [B,seq,H]; rope = (cos, sin) tables [npos, d/2] f32 or None; weight/bias/ln_* as for
    ttt_linear_forward_raw.  Returns (output, weight_out, bias_out[, weight_ckpt, bias_ckpt][, TTTInputsInner]):
    the last item, with save_inputs, holds the operands as the kernel used them (what the backward needs)."""
    B, seq, H, d = xq.shape
    io = xq.dtype
    xq = _need(xq, (B, seq, H, d), io, "xq")
    xk = _need(xk, (B, seq, H, d), io, "xk")
    xv = _need(xv, (B, seq, H, d), io, "xv")
    lg = _need(lr_logits, (B, seq, H), io, "lr_logits")
    lb = _need(lr_bias.reshape(-1), (H,), torch.float32, "lr_bias")
    ti = _need(token_idx, (mini_batch,), torch.float32, "token_idx")
    lti = _need(learnable_token_idx, (mini_batch,), torch.float32, "learnable_token_idx")
    per_batch = weight.dim() == 4
    W0 = _need(weight, (B, H, d, d) if per_batch else (H, d, d), torch.float32, "weight")
    b0 = _need(bias, (B, H, d) if per_batch else (H, d), torch.float32, "bias")
    gam = _need(ln_weight, (H, d), torch.float32, "ln_weight")
    bet = _need(ln_bias, (H, d), torch.float32, "ln_bias")
    null = C.c_void_p(None)
    cos = sin = None
    if rope is not None:
        cos = _need(rope[0], (rope[0].shape[0], d // 2), torch.float32, "rope cos")
        sin = _need(rope[1], (rope[0].shape[0], d // 2), torch.float32, "rope sin")
        last = (pos_offset + seq - 1) if pos_wrap == 0 else min(pos_wrap - 1, pos_offset + seq - 1)
        if last >= cos.shape[0]:
            raise _lib.TttError(_lib.TTT_ERR_SHAPE, "rope table shorter than the positions used")
    dev = xq.device
    desc = TttDesc(B, H, seq, d, mini_batch, eps, checkpoint_interval, _io_dtype(xq), 1 if per_batch else 0, 0,
                   int(packed_checkpoints), 0)
    check(lib().ttt_linear_fwd_fused_inputs_supported(C.byref(desc), pos_wrap, 0 if rope is None else 1))
    out = torch.empty((B, H, seq, d), dtype=io, device=dev)
    W_out = torch.empty((B, H, d, d), dtype=torch.float32, device=dev)
    b_out = torch.empty((B, H, d), dtype=torch.float32, device=dev)
    Wc = bc = None
    if want_checkpoints:
        n = int(lib().ttt_linear_num_checkpoints(C.byref(desc)))
        Wc = torch.empty((B, H, n, d, d), dtype=torch.float32, device=dev)
        bc = torch.empty((B, H, n, d), dtype=torch.float32, device=dev)
    q = k = v = lr = te = None
    if save_inputs:
        q, k, v = (torch.empty((B, H, seq, d), dtype=io, device=dev) for _ in range(3))
        lr = torch.empty((B, H, seq), dtype=io, device=dev)
        te = torch.empty(seq, dtype=torch.float32, device=dev)
    opt = lambda t: null if t is None else _ptr(t)
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    with torch.cuda.device(dev):
        check(lib().ttt_linear_fwd_fused_inputs(
            C.byref(desc), _ptr(xq), _ptr(xk), _ptr(xv), _ptr(lg), _ptr(lb), C.c_float(base_lr), _ptr(ti), _ptr(lti),
            opt(cos), opt(sin), pos_offset, pos_wrap, _ptr(W0), _ptr(b0), _ptr(gam), _ptr(bet), _ptr(out), _ptr(W_out),
            _ptr(b_out), opt(Wc), opt(bc), opt(q), opt(k), opt(v), opt(lr), opt(te), stream))
    res = [out, W_out, b_out]
    if want_checkpoints:
        res += [Wc, bc]
    if save_inputs:
        res.append(TTTInputsInner(Qkv(q, k, v), te, lr))
    return tuple(res)


def layer_epilogue_raw(inner_out, post_norm_weight, post_norm_bias, gate=None, eps: float = 1e-6):
    """One call of ttt_layer_epilogue: head merge + post_norm LayerNorm (+ tanh-GELU gate) of
    TTT::forward (rust/layer/src/ttt.rs:285-297).  inner_out [B,H,seq,d] -> [B,seq,H*d]."""
    B, H, seq, d = inner_out.shape
    io = inner_out.dtype
    x = _need(inner_out, (B, H, seq, d), io, "inner_out")
    g = _need(post_norm_weight, (H * d,), torch.float32, "post_norm_weight")
    b = _need(post_norm_bias, (H * d,), torch.float32, "post_norm_bias")
    gt = None if gate is None else _need(gate, (B, seq, H * d), io, "gate")
    out = torch.empty((B, seq, H * d), dtype=io, device=x.device)
    desc = TttDesc(B, H, seq, d, 1, eps, 1, _io_dtype(x), 0, 0)
    stream = C.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
    with torch.cuda.device(x.device):
        check(lib().ttt_layer_epilogue(C.byref(desc), _ptr(x), _ptr(g), _ptr(b), C.c_float(eps),
                                       C.c_void_p(None) if gt is None else _ptr(gt), _ptr(out), stream))
    return out
