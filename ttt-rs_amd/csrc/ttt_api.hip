// C ABI of the MI355X fused TTT inner loop: argument checks and kernel dispatch.
// Declarations and the reference interfaces they replace: include/ttt_mi355x.h.
#include "../../include/ttt_mi355x.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <vector>

#include "ttt_engine_fwd.hip.h"
#include "ttt_layer_io.hip.h"
#include "ttt_linear_bwd.hip.h"
#include "ttt_linear_bwd_mw.hip.h"
#include "ttt_linear_bwd_pair.hip.h"
#include "ttt_linear_bwd_rr.hip.h"
#include "ttt_linear_fwd.hip.h"
#include "ttt_linear_fwd_mw.hip.h"
#include "ttt_linear_fwd_sk.hip.h"
#include "ttt_mlp_bwd.hip.h"
#include "ttt_mlp_fwd_cl2.hip.h"
#include "ttt_mlp_fwd_rr.hip.h"
#include "ttt_mlpn_fwd.hip.h"
#include "ttt_selftest.hip.h"

// Scratch of ttt_mlp_bwd_static (file scope, outside any namespace so that HIP_SYMBOL names it plainly).
static __device__ __align__(256) unsigned char ttt_mlp_bwd_scratch_mem[TTT_MLP_BWD_STATIC_MAX_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_common(const ttt_desc* d) {
  if (d == nullptr) return fail(TTT_ERR_NULL, "desc is NULL");
  if (d->batch <= 0 || d->heads <= 0 || d->seq <= 0 || d->head_dim <= 0 || d->mini_batch <= 0)
    return fail(TTT_ERR_SHAPE, "batch/heads/seq/head_dim/mini_batch must be positive");
  if (d->seq % d->mini_batch != 0)
    return fail(TTT_ERR_SHAPE, "seq (%d) must be a multiple of mini_batch (%d)", d->seq, d->mini_batch);
  if (d->checkpoint_interval < 1)
    return fail(TTT_ERR_SHAPE, "checkpoint_interval must be >= 1 (got %d)", d->checkpoint_interval);
  if (d->io_dtype != TTT_F32 && d->io_dtype != TTT_BF16)
    return fail(TTT_ERR_UNSUPPORTED, "io_dtype %d is neither TTT_F32 nor TTT_BF16", d->io_dtype);
  if (!(d->eps > 0.f)) return fail(TTT_ERR_SHAPE, "eps must be positive");
  if (d->checkpoint_format != TTT_CKPT_F32 && d->checkpoint_format != TTT_CKPT_PACKED &&
      d->checkpoint_format != TTT_CKPT_FACTORS)
    return fail(TTT_ERR_SHAPE, "checkpoint_format %d is none of TTT_CKPT_F32, TTT_CKPT_PACKED, TTT_CKPT_FACTORS",
                d->checkpoint_format);
  if (d->seq_stride != 0 && d->seq_stride < d->seq)
    return fail(TTT_ERR_SHAPE, "seq_stride (%d) must be 0 or >= seq (%d)", d->seq_stride, d->seq);
  if ((int64_t)d->batch * d->heads > 0x7fffffffLL)
    return fail(TTT_ERR_SHAPE, "batch*heads exceeds the grid limit");
  return TTT_OK;
}

// The checkpoint format a desc stands for after the one substitution the library makes: update factors share the W
// checkpoint buffer with the final state, which takes two or more mini-batches' worth of it, so a sequence of a
// single mini-batch is saved packed.  Forward and backward both decide through this function.
int ckpt_format_of(const ttt_desc* d) {
  if (d->checkpoint_format == TTT_CKPT_FACTORS && d->seq / d->mini_batch < 2) return TTT_CKPT_PACKED;
  return d->checkpoint_format;
}
// What TTT_CKPT_FACTORS needs of a desc (0 = fine); the same for the forward that writes and the backward that reads.
int check_factors(const ttt_desc* d) {
  if (d->io_dtype != TTT_BF16 || d->checkpoint_interval != 1 || d->head_dim > 96 ||
      (d->kernel_hint & TTT_HINT_LDS_TILES) != 0)
    return fail(TTT_ERR_UNSUPPORTED,
                "update-factor checkpoints need bf16 I/O, checkpoint_interval 1, head_dim <= 96 and the "
                "register-resident kernels");
  return TTT_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int hip_status(hipError_t e, const char* what) {
  if (e == hipSuccess) return TTT_OK;
  return fail(TTT_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

// up to ttt::kMaxProblems argument blocks as one kernel argument (unused slots zero)
template <class A>
ttt::Problems<A> pack_of(const A* probs, unsigned n) {
  ttt::Problems<A> P{};
  for (unsigned i = 0; i < n && i < (unsigned)ttt::kMaxProblems; ++i) P.p[i] = probs[i];
  return P;
}

// whether any problem of a launch asks the kernel to form its operands as x + projections (LinearFwdArgs::xin)
bool any_input_sums(const ttt::LinearFwdArgs* probs, unsigned ny) {
  for (unsigned i = 0; i < ny; ++i)
    if (probs[i].xin != nullptr) return true;
  return false;
}

// ---- TTT-Linear forward, head_dim 32/64: kernel choice --------------------------------------
// A (batch, head) unit is a strictly sequential chain of mini-batches, so the launch is latency
// bound until there are more units than SIMDs.  Few units: split each unit over several waves
// (skewed workgroup kernel).  Many units: one wave per unit (no exchange at all).
// desc.kernel_hint (low byte) = 1 | 2 | 4 overrides the number of waves per unit (tuning / tests).
int device_cus(int* cus);

// ctl_wave: f32 I/O, one feature tile per wave, whole mini-batches, a CU per workgroup: the variant with a control
// wave that copies the operands global -> LDS, so that the compute waves issue no loads (same bits; config-2 forward
// 246 -> 216 us, with packed checkpoints 278 -> 250 us)
template <class T, int D, int NW>
int launch_linear_fwd_nw(const ttt::LinearFwdArgs* probs, unsigned ny, hipStream_t s, bool own_loads = false,
                         bool ctl_wave = false) {
  const ttt::LinearFwdArgs& a = probs[0];
  const bool sums = any_input_sums(probs, ny);
  const auto P = pack_of(probs, ny);
  if constexpr (sizeof(typename ttt::Io<T>::elem) == 4 && NW == D / 16 && NW > 1) {
    if (ctl_wave && a.K == 16 && !sums) {
      hipLaunchKernelGGL((ttt::ttt_linear_fwd_dma_kernel<T, D, NW, 2>), dim3((unsigned)(a.B * a.H), ny), dim3(64 * (NW + 1)), 0, s, P);
      return hip_status(hipGetLastError(), "ttt_linear_fwd launch");
    }
  }
  // mini-batches prefetched ahead, in registers (f32 fragments are twice as large: the one-wave f32 kernel, which
  // holds the whole state and all rows in one wave, has registers for one mini-batch ahead only)
  constexpr int PF = (NW == 1 && sizeof(typename ttt::Io<T>::elem) == 4) ? 1 : 2;
  const dim3 grid((unsigned)(a.B * a.H), ny), block(64 * NW);
  // the variants that save update factors exist for bf16 I/O only (prepare_linear_fwd lets no other desc ask)
  constexpr bool can_fac = sizeof(typename ttt::Io<T>::elem) == 2;
  const bool fac = can_fac && a.ckpt_packed == ttt::kCkptFactors;
  if constexpr (NW == 1) {
    if constexpr (can_fac) {
      if (fac) {
        if (a.K == 16)
          hipLaunchKernelGGL((ttt::ttt_linear_fwd_mw_kernel<T, D, 1, PF, true, true>), grid, block, 0, s, P);
        else
          hipLaunchKernelGGL((ttt::ttt_linear_fwd_mw_kernel<T, D, 1, PF, false, true>), grid, block, 0, s, P);
        return hip_status(hipGetLastError(), "ttt_linear_fwd launch");
      }
    }
    if (a.K == 16)
      hipLaunchKernelGGL((ttt::ttt_linear_fwd_mw_kernel<T, D, 1, PF, true>), grid, block, 0, s, P);
    else
      hipLaunchKernelGGL((ttt::ttt_linear_fwd_mw_kernel<T, D, 1, PF, false>), grid, block, 0, s, P);
  } else {
    constexpr int NWS = NW > 1 ? NW : 2;  // the skewed kernel needs at least two waves
    // bf16, head_dim 64, two waves per unit: the variant in which a wave loads only the features it owns and the
    // full rows cross LDS (same bits).  Measured on MI355X (seq 2048): 24 units 117 us against 114 us, 252 units
    // 120 against 120, 384 units 129 - 139 against 137 - 146: it pays once two workgroups share a CU's load path.
    if constexpr (can_fac && NWS == 2 && D == 64) {
      if (sums) {  // operands formed as x + projections (a layer of a stack); no checkpoints in that mode
        if (a.K == 16)
          hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, true, false, 2>), grid, block, 0, s, P);
        else
          hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, false, false, 2>), grid, block, 0, s, P);
        return hip_status(hipGetLastError(), "ttt_linear_fwd launch");
      }
      if (own_loads) {
        if (fac) {
          if (a.K == 16)
            hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, true, true, true>), grid, block, 0, s, P);
          else
            hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, false, true, true>), grid, block, 0, s, P);
        } else if (a.K == 16) {
          hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, true, false, true>), grid, block, 0, s, P);
        } else {
          hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, false, false, true>), grid, block, 0, s, P);
        }
        return hip_status(hipGetLastError(), "ttt_linear_fwd launch");
      }
    }
    if constexpr (can_fac) {
      if (fac) {
        if (a.K == 16)
          hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, true, true>), grid, block, 0, s, P);
        else
          hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, false, true>), grid, block, 0, s, P);
        return hip_status(hipGetLastError(), "ttt_linear_fwd launch");
      }
    }
    if (a.K == 16)
      hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, true>), grid, block, 0, s, P);
    else
      hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NWS, PF, false>), grid, block, 0, s, P);
  }
  return hip_status(hipGetLastError(), "ttt_linear_fwd launch");
}

template <class T, int D>
int launch_linear_fwd(const ttt::LinearFwdArgs* probs, int hint, unsigned ny, hipStream_t s) {
  const int waves_hint = hint & TTT_HINT_WAVES_MASK;
  const ttt::LinearFwdArgs& a = probs[0];
  constexpr bool f32 = sizeof(typename ttt::Io<T>::elem) == 4;
  // bf16 I/O: one or two waves per unit.  A four-wave bf16 variant (one feature tile per wave) is not offered: it
  // was never faster than two, and its output LayerNorm came out wrong for one mini-batch in three of the
  // branch-free passes (the k = 16 matrix instruction that adds the causal correction onto the k = 32 products).
  constexpr int max_nw = f32 ? D / 16 : (D / 16 < 2 ? D / 16 : 2);
  const long units = (long)a.B * a.H * ny;
  int nw = waves_hint;
  if (nw <= 0) {
    // measured on MI355X (256 CUs x 4 SIMDs): bf16 is VALU-latency bound and likes 2 waves per unit
    // up to ~2 units per CU; f32 is MFMA bound (16x16x4 f32) and likes 4 until the CUs are shared
    if (f32)
      nw = units <= 256 ? 4 : (units <= 512 ? 2 : 1);
    else
      nw = units <= 512 ? 2 : 1;
  }
  if (nw > max_nw) nw = max_nw;
  if constexpr (!f32 && D == 64) {
    if (any_input_sums(probs, ny)) nw = 2;  // the kernel that forms x + projections is the two-wave one
  }
  // f32 I/O with a CU per workgroup: the control-wave variant (TTT_HINT_ALL_LOADS keeps the loads in the compute waves)
  bool ctl_wave = false;
  if constexpr (f32) {
    int cus = 0;
    if ((hint & TTT_HINT_ALL_LOADS) == 0 && device_cus(&cus) == TTT_OK) ctl_wave = units <= cus;
  }
  if constexpr (max_nw >= 4) {
    if (nw >= 4) return launch_linear_fwd_nw<T, D, 4>(probs, ny, s, false, ctl_wave);
  }
  // a launch that puts two workgroups on a CU, or a caller that asks for it
  const bool own_loads = units > 256 ? (hint & TTT_HINT_ALL_LOADS) == 0 : (hint & TTT_HINT_OWN_LOADS) != 0;
  if (nw >= 2) return launch_linear_fwd_nw<T, D, 2>(probs, ny, s, own_loads, ctl_wave && max_nw == 2);
  return launch_linear_fwd_nw<T, D, 1>(probs, ny, s);
}

// ---- TTT-Linear forward, head_dim 96/128: the same register-resident skewed kernel with two
// feature tiles per wave (3 waves at d = 96, 4 at d = 128; one tile per wave was measured slower for
// every shape tried: twice the waves exchange twice the row sums).  The LDS-tile kernel stays
// available through TTT_HINT_LDS_TILES.
template <class T, int D>
int launch_linear_fwd_wide(const ttt::LinearFwdArgs* probs, unsigned ny, hipStream_t s) {
  const ttt::LinearFwdArgs& a = probs[0];
  const auto P = pack_of(probs, ny);
  constexpr int NW = D / 32;
  constexpr bool f32 = sizeof(typename ttt::Io<T>::elem) == 4;
  constexpr int PF = f32 ? 1 : 2;  // f32 fragments are twice as large: prefetch one mini-batch ahead
  const dim3 grid((unsigned)(a.B * a.H), ny), block(64 * NW);
  if constexpr (!f32 && D == 128) {
    if (any_input_sums(probs, ny)) {
      if (a.K == 16)
        hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NW, PF, true, false, 2>), grid, block, 0, s, P);
      else
        hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NW, PF, false, false, 2>), grid, block, 0, s, P);
      return hip_status(hipGetLastError(), "ttt_linear_fwd launch");
    }
  }
  if constexpr (!f32 && D == 96) {
    if (a.ckpt_packed == ttt::kCkptFactors) {
      if (a.K == 16)
        hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NW, PF, true, true>), grid, block, 0, s, P);
      else
        hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NW, PF, false, true>), grid, block, 0, s, P);
      return hip_status(hipGetLastError(), "ttt_linear_fwd launch");
    }
  }
  if (a.K == 16)
    hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NW, PF, true>), grid, block, 0, s, P);
  else
    hipLaunchKernelGGL((ttt::ttt_linear_fwd_sk_kernel<T, D, NW, PF, false>), grid, block, 0, s, P);
  return hip_status(hipGetLastError(), "ttt_linear_fwd launch");
}

// More than the default 64 KiB of LDS per workgroup has to be requested per kernel and device.  Done once:
// one bit per device ordinal and kernel (the kernel is a template argument, so every kernel has its own mask).
template <auto Kern>
int opt_in_lds(size_t bytes) {
  static std::atomic<uint64_t> done{0};
  int dev = 0;
  int rc = hip_status(hipGetDevice(&dev), "hipGetDevice");
  if (rc != TTT_OK) return rc;
  const uint64_t bit = (dev >= 0 && dev < 64) ? (uint64_t)1 << dev : 0;
  if (bit != 0 && (done.load(std::memory_order_acquire) & bit) != 0) return TTT_OK;
  rc = hip_status(hipFuncSetAttribute(reinterpret_cast<const void*>(Kern),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes),
                  "hipFuncSetAttribute(LDS size)");
  if (rc == TTT_OK) done.fetch_or(bit, std::memory_order_release);
  return rc;
}

template <class T, int D, int MT = 1, bool BF = false>
int launch_linear_fwd_lds(const ttt::LinearFwdArgs* probs, unsigned ny, hipStream_t s) {
  const ttt::LinearFwdArgs& a = probs[0];
  constexpr auto kern = ttt::ttt_linear_fwd_lds_kernel<T, D, MT, BF>;
  constexpr size_t bytes = ttt::LinFwdLds<D, MT>::BYTES;
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)(a.B * a.H), ny), dim3(256 * MT), bytes, s, pack_of(probs, ny));
  return hip_status(hipGetLastError(), "ttt_linear_fwd (LDS kernel) launch");
}

template <class T, int D>
int launch_mlp_fwd(const ttt::MlpFwdArgs* probs, unsigned ny, hipStream_t s) {
  const ttt::MlpFwdArgs& a = probs[0];
  constexpr auto kern = ttt::ttt_mlp_fwd_kernel<T, D>;
  constexpr size_t bytes = ttt::MlpLds<D>::BYTES;
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)(a.B * a.H), ny), dim3(512), bytes, s, pack_of(probs, ny));
  return hip_status(hipGetLastError(), "ttt_mlp_fwd launch");
}

// register-resident kernel (d <= 96, bf16 operands on the matrix cores)
template <class T, int D>
int launch_mlp_fwd_rr(const ttt::MlpFwdArgs* probs, unsigned ny, hipStream_t s) {
  const ttt::MlpFwdArgs& a = probs[0];
  constexpr auto kern = ttt::ttt_mlp_fwd_rr_kernel<T, D>;
  constexpr size_t bytes = ttt::MlpRrLds<D, sizeof(typename ttt::Io<T>::elem)>::BYTES;
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)(a.B * a.H), ny), dim3(512), bytes, s, pack_of(probs, ny));
  return hip_status(hipGetLastError(), "ttt_mlp_fwd (register-resident kernel) launch");
}

// bf16 I/O, head_dim 128 (and 96 when there are few units): a pair of workgroups per (batch, head); the exchange flags
// live in W2_out, which is zeroed first (a fill kernel, not a memset node).
// The two workgroups of a pair wait for each other, so both must be resident: a workgroup fills a CU (LDS,
// registers), hence no launch may hold more workgroups than the device has CUs.  The units are independent, so
// more units than that go in several launches on the stream.  Several problems travel together while they fit
// that limit, otherwise one after the other.
int device_cus(int* cus) {
  int dev = 0;
  int rc = hip_status(hipGetDevice(&dev), "hipGetDevice");
  if (rc != TTT_OK) return rc;
  return hip_status(hipDeviceGetAttribute(cus, hipDeviceAttributeMultiprocessorCount, dev), "hipDeviceGetAttribute(CU count)");
}

template <int D>
int launch_mlp_fwd_cl2(const ttt::MlpFwdArgs* probs, int n, hipStream_t s) {
  constexpr auto kern = ttt::ttt_mlp_fwd_cl2_kernel<ttt::BF16, D>;
  constexpr size_t bytes = ttt::MlpCl2Lds<D, 2>::BYTES;
  constexpr unsigned threads = 64 * (D / 16);
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  int cus = 0;
  rc = device_cus(&cus);
  if (rc != TTT_OK) return rc;
  const size_t units = (size_t)probs[0].B * probs[0].H, nz = units * D * (4 * D);
  for (int p = 0; p < n; ++p)
    if (!probs[p].exchange_cleared)
      hipLaunchKernelGGL(ttt::ttt_fill_zero_kernel, dim3((unsigned)((nz + 255) / 256)), dim3(256), 0, s, probs[p].W2, nz);
  const size_t per_launch = (size_t)(cus / 16 > 0 ? cus / 16 : 1) * 8;  // groups of 16 workgroups = 8 units
  const size_t wg_per_problem = ((units + 7) / 8) * 16;
  int together = (int)((size_t)cus / wg_per_problem);  // whole problems that fit the device at once
  if (together > ttt::kMaxProblems) together = ttt::kMaxProblems;
  for (int p = 0; p < n;) {
    if (together >= 2 && n - p >= 2) {
      const int cnt = n - p < together ? n - p : together;
      hipLaunchKernelGGL(kern, dim3((unsigned)wg_per_problem, (unsigned)cnt), dim3(threads), bytes, s, pack_of(probs + p, (unsigned)cnt));
      p += cnt;
      continue;
    }
    ttt::MlpFwdArgs a = probs[p];
    for (size_t base = 0; base < units; base += per_launch) {
      const size_t cnt = units - base < per_launch ? units - base : per_launch;
      a.unit_base = (int)base;
      hipLaunchKernelGGL(kern, dim3((unsigned)(((cnt + 7) / 8) * 16)), dim3(threads), bytes, s, pack_of(&a, 1));
    }
    ++p;
  }
  return hip_status(hipGetLastError(), "ttt_mlp_fwd (two-CU kernel) launch");
}

// Whether ttt_mlp_fwd runs the two-CU kernel for this desc and this many problems of its shape in one dispatch:
// bf16 I/O without TTT_HINT_LDS_TILES; head_dim 128 always (the state does not fit one CU); head_dim 96 on request
// (TTT_HINT_TWO_CU), for a single problem with at most half as many units as the device has CUs.  Measured at
// B = 8, H = 16, seq 2048 (128 units on 256 CUs): 0.83 - 0.85 ms on pairs against 0.86 ms on single CUs -- the
// exchange through global memory costs what halving each CU's share of the hidden axis saves -- so it is not the default.
int uses_two_cu_mlp(const ttt_desc* d, int n_problems, bool* yes) {
  *yes = false;
  if (d->io_dtype == TTT_F32 || (d->kernel_hint & TTT_HINT_LDS_TILES) != 0) return TTT_OK;
  if (d->head_dim == 128) {
    *yes = true;
    return TTT_OK;
  }
  if (d->head_dim != 96 || n_problems != 1 || (d->kernel_hint & TTT_HINT_TWO_CU) == 0) return TTT_OK;
  int cus = 0;
  const int rc = device_cus(&cus);
  if (rc != TTT_OK) return rc;
  *yes = 2 * (int64_t)d->batch * d->heads <= cus;
  return TTT_OK;
}

template <class T, int D, int MT = 1, bool WG = false, bool DG = false, bool BF = false>
int launch_linear_bwd(const ttt::LinearBwdArgs& a, unsigned grid, hipStream_t s) {
  constexpr auto kern = ttt::ttt_linear_bwd_kernel<T, D, MT, WG, DG, BF>;
  constexpr size_t bytes = ttt::BwdLds<D, MT, WG, DG>::BYTES;
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256 * MT), bytes, s, a);
  return hip_status(hipGetLastError(), "ttt_linear_bwd launch");
}

// bf16 I/O, one checkpoint per mini-batch: one wave per (batch, head), state gradient in registers
template <int D, bool PK = false>
int launch_linear_bwd_rr(const ttt::LinearBwdArgs& a, unsigned grid, hipStream_t s) {
  constexpr auto kern = ttt::ttt_linear_bwd_rr_kernel<ttt::BF16, D, PK>;
  constexpr size_t bytes = ttt::LinBwdRrLds<D, PK>::BYTES;
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64), bytes, s, a);
  return hip_status(hipGetLastError(), "ttt_linear_bwd (register-resident kernel) launch");
}

// one checkpoint per mini-batch, NW waves per (batch, head): feature axis split, exchanges through LDS
template <class T, int D, int NW, bool PK = false, bool FM = false>
int launch_linear_bwd_mw(const ttt::LinearBwdArgs& a, unsigned grid, hipStream_t s) {
  constexpr size_t bytes = ttt::LinBwdMwLds<D, NW, sizeof(typename ttt::Io<T>::elem), PK, FM>::BYTES;
  // opaque checkpoints (the training path): a variant for whole mini-batches of 16 tokens
  if constexpr (PK) {
    if (a.K == 16) {
      constexpr auto kern16 = ttt::ttt_linear_bwd_mw_kernel<T, D, NW, PK, FM, true>;
      int rc = opt_in_lds<kern16>(bytes);
      if (rc != TTT_OK) return rc;
      hipLaunchKernelGGL(kern16, dim3(grid), dim3(64 * NW), bytes, s, a);
      return hip_status(hipGetLastError(), "ttt_linear_bwd (multi-wave register-resident kernel) launch");
    }
  }
  constexpr auto kern = ttt::ttt_linear_bwd_mw_kernel<T, D, NW, PK, FM>;
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * NW), bytes, s, a);
  return hip_status(hipGetLastError(), "ttt_linear_bwd (multi-wave register-resident kernel) launch");
}

// f32 I/O, one checkpoint per mini-batch, two workgroups per (batch, head): workgroups b and b + 8 of every 16 share a unit
template <int D, bool PK>
int launch_linear_bwd_pair(const ttt::LinearBwdPairArgs& pa, hipStream_t s) {
  constexpr size_t bytes = ttt::LinBwdPair<D, PK>::BYTES;
  const unsigned units = (unsigned)(pa.a.B * pa.a.H), grid = (units + 7) / 8 * 16;
  if (pa.a.K == 16) {
    constexpr auto kern16 = ttt::ttt_linear_bwd_pair_kernel<D, PK, true>;
    int rc = opt_in_lds<kern16>(bytes);
    if (rc != TTT_OK) return rc;
    hipLaunchKernelGGL(kern16, dim3(grid), dim3(64 * (D / 16 + 1)), bytes, s, pa);
    return hip_status(hipGetLastError(), "ttt_linear_bwd_ws (two workgroups per unit) launch");
  }
  constexpr auto kern = ttt::ttt_linear_bwd_pair_kernel<D, PK, false>;
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * (D / 16 + 1)), bytes, s, pa);
  return hip_status(hipGetLastError(), "ttt_linear_bwd_ws (two workgroups per unit) launch");
}

template <class T, int D, bool BF, bool PIPE>
int launch_mlp_bwd_as(const ttt::MlpBwdArgs& a, hipStream_t s) {
  constexpr auto kern = ttt::ttt_mlp_bwd_kernel<T, D, BF, PIPE>;
  constexpr size_t bytes = ttt::MlpBwdLds<D>::BYTES;
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  // two workgroups per unit: workgroups b and b + 8 of every 16 share a unit
  const unsigned units = (unsigned)(a.B * a.H), grid = PIPE ? (units + 7) / 8 * 16 : units;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), bytes, s, a);
  return hip_status(hipGetLastError(), "ttt_mlp_bwd launch");
}
template <class T, int D, bool BF = false>
int launch_mlp_bwd(const ttt::MlpBwdArgs& a, hipStream_t s) {
  static_assert(ttt::MlpBwdPipe<D>::FLOATS == 4 * D * 4 * D + ttt::kMlpBwdSharedTiles * 16 * 4 * D + 2 * ((48 * D + 4 * 256 + 16 + D + 3) / 4 * 4),
                "MlpBwdWs computes the same size");
  if (a.pipe != nullptr) return launch_mlp_bwd_as<T, D, BF, true>(a, s);
  return launch_mlp_bwd_as<T, D, BF, false>(a, s);
}

// Which TTT-Linear backward kernel serves a desc (and whether one does).
// One checkpoint per mini-batch: the register-resident kernels (the state entering a mini-batch is read, not
// re-simulated).  Waves per (batch, head): f32 products are bound by the matrix pipe, so the feature axis is
// always split; bf16 runs one wave per unit when there are more units than two per CU and the split kernel
// otherwise.  Coarser checkpoints (states re-simulated from the last checkpoint) or TTT_HINT_LDS_TILES: the
// LDS-tile kernel, head_dim <= 64.  desc.kernel_hint's low byte overrides the number of waves.
struct LinearBwdChoice {
  enum Kind { LDS, REG } kind;
  int waves;
  // LDS-tile kernel only: the state gradient lives in the d_W0 buffer / the state is read in place from its checkpoint
  bool dw_global = false, w_global = false;
};
int choose_linear_bwd(const ttt_desc* d, LinearBwdChoice* ch) {
  int rc = ttt_linear_supported(d);
  if (rc != TTT_OK) return rc;
  const int D = d->head_dim;
  const bool f32 = d->io_dtype == TTT_F32;
  if (d->checkpoint_format == TTT_CKPT_FACTORS) {
    rc = check_factors(d);
    if (rc != TTT_OK) return rc;
  }
  const bool packed = ckpt_format_of(d) == TTT_CKPT_PACKED;
  const bool factors = ckpt_format_of(d) == TTT_CKPT_FACTORS;
  if (d->mini_batch > 16) {
    // two tiles of token rows: the LDS-tile kernel, any checkpoint interval, f32 row-major checkpoints
    if (packed || factors)
      return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_bwd: mini_batch %d > 16 reads f32 row-major checkpoints only", d->mini_batch);
    ch->kind = LinearBwdChoice::LDS;
    ch->waves = 8;
    return TTT_OK;
  }
  const bool want_lds = (d->kernel_hint & TTT_HINT_LDS_TILES) != 0 && D <= 64;
  if (packed && (d->checkpoint_interval != 1 || want_lds))
    return fail(TTT_ERR_UNSUPPORTED, "packed checkpoints need checkpoint_interval 1 and the register-resident kernels");
  if (d->checkpoint_interval == 1 && !want_lds) {
    if (f32 && D == 128) {
      // the f32 staging of the register-resident kernel does not fit a CU at head_dim 128: the LDS-tile kernel with
      // the state read in place from the (row-major) checkpoints and the state gradient kept in d_W0
      if (packed) return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_bwd: head_dim 128 with f32 I/O reads f32 row-major checkpoints only");
      ch->kind = LinearBwdChoice::LDS;
      ch->waves = 4;
      ch->w_global = ch->dw_global = true;
      return TTT_OK;
    }
    int waves = d->kernel_hint & TTT_HINT_WAVES_MASK;
    const long units = (long)d->batch * d->heads;
    // bf16 at head_dim 64 between 257 and 512 units, f32 row-major checkpoints: two waves per unit.  Four waves per
    // unit put eight waves on the four SIMDs of every CU that hosts two workgroups; with two, every wave keeps a SIMD
    // to itself (measured at 384 units: 544 us against 606 us; at 192 units 513 against 392).  With packed states or
    // update factors the four-wave kernel stays ahead at 384 units as well (456 against 468 us, 440 against 473 us),
    // so there two waves are a matter of the hint.
    const bool two = !f32 && D == 64 && units > 256 && units <= 512 && !packed && !factors;
    if (waves == 0) waves = two ? 2 : (f32 || D > 64 || units <= 512) ? 4 : 1;
    // the walk back of the state exists in the feature-split kernel only
    if (factors && (waves < 2 || (waves == 2 && D != 64))) waves = 4;
    ch->kind = LinearBwdChoice::REG;
    ch->waves = waves;
    return TTT_OK;
  }
  // coarser checkpoints: the state is re-simulated in LDS.  head_dim 96: with the state gradient in d_W0 the rest
  // fits; head_dim 128: the state alone leaves too little LDS for the tiles of a stage
  if (D > 96)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_bwd: head_dim %d needs checkpoint_interval 1 (got %d)", D,
                d->checkpoint_interval);
  ch->kind = LinearBwdChoice::LDS;
  ch->waves = 4;
  ch->dw_global = D == 96;
  return TTT_OK;
}

// dst = src, or zeros when src is null (a kernel, not a memcpy/memset node: capturable)
__global__ void ttt_copy_or_zero_kernel(float* dst, const float* src, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src ? src[i] : 0.f;
}
void copy_or_zero(float* dst, const float* src, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(ttt_copy_or_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, dst, src, n);
}

// Whether the TTT-MLP reverse scan spreads every unit over two workgroups (producer and consumer, see
// ttt_mlp_bwd_kernel): when every pair can have two CUs of its own.  A function of the desc alone, because the size of
// the workspace follows from it; the launch checks the device's CU count on top.
constexpr int kMlpBwdPipeMaxUnits = 128;
bool mlp_bwd_pipe(const ttt_desc* d) {
  return (int64_t)d->batch * d->heads <= kMlpBwdPipeMaxUnits && !(d->kernel_hint & TTT_HINT_ONE_WORKGROUP);
}

// float offsets of the pieces of the ttt_mlp_bwd workspace
struct MlpBwdWs {
  size_t W1, W2, b1, b2, G1s, G2s, mt, pipe, flags, total;
  explicit MlpBwdWs(const ttt_desc* d) {
    const size_t U = (size_t)d->batch * d->heads, D = d->head_dim, M = 4 * D, N = d->seq / d->mini_batch;
    W1 = 0;
    W2 = W1 + U * D * M;
    b1 = W2 + U * M * D;
    b2 = b1 + U * M;
    G1s = b2 + U * D;
    G2s = G1s + U * N * 16 * M;
    mt = G2s + U * N * 16 * D;
    total = mt + U * ttt::kMlpBwdMTiles * 16 * M;
    pipe = flags = total;
    if (mlp_bwd_pipe(d)) {
      // the same arithmetic as ttt::MlpBwdPipe<D>::FLOATS
      const size_t xb = (48 * D + 4 * 256 + 16 + D + 3) / 4 * 4;
      const size_t per_unit = 2 * D * M + ttt::kMlpBwdSharedTiles * 16 * M + 2 * xb + 2 * D * M;
      flags = pipe + U * per_unit;
      total = flags + U * ttt::kMlpBwdPipeFlagWords;
    }
  }
};

template <class T>
void launch_epilogue(const ttt::LayerEpilogueArgs& a, int nc, dim3 grid, hipStream_t s) {
  switch (nc) {
    case 1: hipLaunchKernelGGL((ttt::ttt_layer_epilogue_kernel<T, 1>), grid, dim3(256), 0, s, a); break;
    case 2: hipLaunchKernelGGL((ttt::ttt_layer_epilogue_kernel<T, 2>), grid, dim3(256), 0, s, a); break;
    default: hipLaunchKernelGGL((ttt::ttt_layer_epilogue_kernel<T, 4>), grid, dim3(256), 0, s, a); break;
  }
}


// ---- built-in scratch of ttt_mlp_bwd_static ------------------------------------------------------
// Device memory that belongs to the library's code object: every GPU the library runs on holds its own
// copy at its own address until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels and fills get the looked-up device address.
constexpr size_t kMlpBwdScratchBytes = TTT_MLP_BWD_STATIC_MAX_BYTES;
constexpr int kMaxDevices = 64;
std::atomic<void*> g_mlp_bwd_scratch[kMaxDevices];

int mlp_bwd_scratch(void** out) {
  int dev = -1;
  int rc = hip_status(hipGetDevice(&dev), "hipGetDevice");
  if (rc != TTT_OK) return rc;
  if (dev < 0 || dev >= kMaxDevices) return fail(TTT_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
  void* p = g_mlp_bwd_scratch[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    // first call on this device (it is the current one): every thread that gets here looks up the same address
    rc = hip_status(hipGetSymbolAddress(&p, HIP_SYMBOL(ttt_mlp_bwd_scratch_mem)), "hipGetSymbolAddress(scratch)");
    if (rc != TTT_OK) return rc;
    if (p == nullptr) return fail(TTT_ERR_HIP, "hipGetSymbolAddress(scratch) returned a null address");
    g_mlp_bwd_scratch[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return TTT_OK;
}

// Whether the forward sweep of a TTT-MLP backward is the register-resident forward (bf16 I/O up to head_dim 96, no
// request for f32 products through TTT_HINT_LDS_TILES): the reverse scan then takes bf16 operands as well.
bool mlp_rr_sweep(const ttt_desc* d) {
  return d->io_dtype != TTT_F32 && d->head_dim <= 96 && !(d->kernel_hint & TTT_HINT_LDS_TILES);
}

// sweep = false: the workspace already holds what the sweep leaves there (ttt_mlp_fwd_saving wrote it)
int mlp_bwd_impl(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                const float* token_eta, const void* lr, const float* gamma, const float* beta,
                const void* d_out, const float* d_W1_out, const float* d_b1_out,
                const float* d_W2_out, const float* d_b2_out, void* d_xq, void* d_xk, void* d_xv,
                float* d_W1, float* d_b1, float* d_W2, float* d_b2, void* d_lr, float* d_token_eta,
                float* d_gamma, float* d_beta, void* workspace, void* stream, bool sweep = true) {
  int rc = ttt_mlp_supported(d);
  if (rc != TTT_OK) return rc;
  if (!xq || !xk || !xv || !W1_0 || !b1_0 || !W2_0 || !b2_0 || !token_eta || !lr || !gamma || !beta ||
      !d_out || !d_xq || !d_xk || !d_xv || !d_W1 || !d_b1 || !d_W2 || !d_b2 || !d_lr || !d_token_eta ||
      !d_gamma || !d_beta || !workspace)
    return fail(TTT_ERR_NULL, "ttt_mlp_bwd: a required pointer is NULL");
  const bool up = d_W1_out || d_b1_out || d_W2_out || d_b2_out;
  if (up && !(d_W1_out && d_b1_out && d_W2_out && d_b2_out))
    return fail(TTT_ERR_NULL, "ttt_mlp_bwd: the four upstream state gradients must all be given or all be NULL");
  if (!aligned16(workspace)) return fail(TTT_ERR_SHAPE, "ttt_mlp_bwd: workspace must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const MlpBwdWs w(d);
  float* ws = static_cast<float*>(workspace);
  const bool f32 = d->io_dtype == TTT_F32;
  const size_t U = (size_t)d->batch * d->heads, D = d->head_dim, M = 4 * D;

  // forward sweep: final state and, per mini-batch, the rank-16 factors of the state update.  bf16 I/O up to
  // head_dim 96: the register-resident forward itself (the factors are then the ones the forward of this step
  // applied, rounded to bf16 as its matrix instructions took them); its output goes to d_xq, which the reverse
  // scan overwrites afterwards.  Otherwise the LDS-tile kernel (f32 products, no output).
  const bool rr_sweep = mlp_rr_sweep(d);
  ttt::MlpFwdArgs fa;
  fa.xq = xq; fa.xk = xk; fa.xv = xv; fa.W1_0 = W1_0; fa.b1_0 = b1_0; fa.W2_0 = W2_0; fa.b2_0 = b2_0;
  fa.token_eta = token_eta; fa.lr = lr; fa.gamma = gamma; fa.beta = beta; fa.out = nullptr;
  fa.W1 = ws + w.W1; fa.b1 = ws + w.b1; fa.W2 = ws + w.W2; fa.b2 = ws + w.b2;
  fa.G1_save = ws + w.G1s; fa.G2_save = ws + w.G2s; fa.unit_base = 0; fa.spin_limit = 1 << 21; fa.exchange_cleared = 0; fa.assume_other_xcd = 0;
  fa.B = d->batch; fa.H = d->heads; fa.seq = d->seq; fa.K = d->mini_batch;
  fa.seq_stride = d->seq_stride > 0 ? d->seq_stride : d->seq;
  fa.n_stages = d->seq / d->mini_batch;
  fa.state_per_batch = d->state_per_batch ? 1 : 0;
  fa.eps = d->eps;
  if (!sweep) {
    rc = TTT_OK;
  } else if (rr_sweep) {
    fa.out = d_xq;
    switch (d->head_dim) {
      case 32: rc = launch_mlp_fwd_rr<ttt::BF16, 32>(&fa, 1, s); break;
      case 64: rc = launch_mlp_fwd_rr<ttt::BF16, 64>(&fa, 1, s); break;
      default: rc = launch_mlp_fwd_rr<ttt::BF16, 96>(&fa, 1, s); break;
    }
  } else
  switch (d->head_dim) {
    case 32: rc = f32 ? launch_mlp_fwd<ttt::F32, 32>(&fa, 1, s) : launch_mlp_fwd<ttt::BF16, 32>(&fa, 1, s); break;
    case 64: rc = f32 ? launch_mlp_fwd<ttt::F32, 64>(&fa, 1, s) : launch_mlp_fwd<ttt::BF16, 64>(&fa, 1, s); break;
    case 96: rc = f32 ? launch_mlp_fwd<ttt::F32, 96>(&fa, 1, s) : launch_mlp_fwd<ttt::BF16, 96>(&fa, 1, s); break;
    default: rc = f32 ? launch_mlp_fwd<ttt::F32, 128>(&fa, 1, s) : launch_mlp_fwd<ttt::BF16, 128>(&fa, 1, s); break;
  }
  if (rc != TTT_OK) return rc;

  // gradient accumulators start from the upstream state gradients (or zero); the reductions over
  // batch / heads start from zero
  copy_or_zero(d_W1, d_W1_out, U * D * M, s);
  copy_or_zero(d_b1, d_b1_out, U * M, s);
  copy_or_zero(d_W2, d_W2_out, U * M * D, s);
  copy_or_zero(d_b2, d_b2_out, U * D, s);
  {
    const size_t hd = (size_t)d->heads * D, nmax = (size_t)d->seq > hd ? (size_t)d->seq : hd;
    hipLaunchKernelGGL(ttt::ttt_fill_zero3_kernel, dim3((unsigned)((nmax + 255) / 256)), dim3(256), 0, s, d_token_eta,
                       (size_t)d->seq, d_gamma, hd, d_beta, hd);
  }
  rc = hip_status(hipGetLastError(), "ttt_mlp_bwd fills");
  if (rc != TTT_OK) return rc;

  ttt::MlpBwdArgs a;
  a.xq = xq; a.xk = xk; a.xv = xv; a.token_eta = token_eta; a.lr = lr; a.gamma = gamma; a.beta = beta;
  a.d_out = d_out; a.G1s = ws + w.G1s; a.G2s = ws + w.G2s; a.W1 = ws + w.W1; a.W2 = ws + w.W2;
  a.b1f = ws + w.b1; a.b2f = ws + w.b2; a.mt = ws + w.mt;
  a.d_xq = d_xq; a.d_xk = d_xk; a.d_xv = d_xv; a.d_W1 = d_W1; a.d_b1 = d_b1; a.d_W2 = d_W2; a.d_b2 = d_b2;
  a.d_lr = d_lr; a.d_token_eta = d_token_eta; a.d_gamma = d_gamma; a.d_beta = d_beta;
  a.B = d->batch; a.H = d->heads; a.seq = d->seq; a.K = d->mini_batch;
  a.seq_stride = fa.seq_stride; a.n_stages = fa.n_stages; a.eps = d->eps;
  a.pipe = nullptr; a.pipe_flags = nullptr; a.spin_limit = 1u << 21; a.agent_release = 0;
  if (mlp_bwd_pipe(d)) {
    // both workgroups of every unit must be resident together: as many CUs as workgroups
    int cus = 0;
    rc = device_cus(&cus);
    if (rc != TTT_OK) return rc;
    if ((int64_t)(U + 7) / 8 * 16 <= cus) {
      a.pipe = ws + w.pipe;
      a.pipe_flags = reinterpret_cast<unsigned*>(ws + w.flags);
      if (d->kernel_hint & TTT_HINT_TEST_LOST_PARTNER) a.spin_limit = 0;
      if (d->kernel_hint & TTT_HINT_TEST_OTHER_XCD) a.agent_release = 1;
      copy_or_zero(ws + w.flags, nullptr, U * ttt::kMlpBwdPipeFlagWords, s);
      rc = hip_status(hipGetLastError(), "ttt_mlp_bwd flag fill");
      if (rc != TTT_OK) return rc;
    }
  }
  // behind the register-resident sweep the scan takes bf16 operands too (the states it walks back through were
  // formed from bf16 operands); TTT_HINT_F32_PRODUCTS keeps the scan's products in f32
  if (rr_sweep && !(d->kernel_hint & TTT_HINT_F32_PRODUCTS)) switch (d->head_dim) {
      case 32: return launch_mlp_bwd<ttt::BF16, 32, true>(a, s);
      case 64: return launch_mlp_bwd<ttt::BF16, 64, true>(a, s);
      default: return launch_mlp_bwd<ttt::BF16, 96, true>(a, s);
    }
  switch (d->head_dim) {
    case 32: return f32 ? launch_mlp_bwd<ttt::F32, 32>(a, s) : launch_mlp_bwd<ttt::BF16, 32>(a, s);
    case 64: return f32 ? launch_mlp_bwd<ttt::F32, 64>(a, s) : launch_mlp_bwd<ttt::BF16, 64>(a, s);
    case 96: return f32 ? launch_mlp_bwd<ttt::F32, 96>(a, s) : launch_mlp_bwd<ttt::BF16, 96>(a, s);
    default: return f32 ? launch_mlp_bwd<ttt::F32, 128>(a, s) : launch_mlp_bwd<ttt::BF16, 128>(a, s);
  }
}

}  // namespace

extern "C" {

const char* ttt_version(void) { return "ttt-mi355x 0.1 (gfx950)"; }

const char* ttt_last_error(void) { return g_err; }

int ttt_linear_supported(const ttt_desc* d) {
  int rc = check_common(d);
  if (rc != TTT_OK) return rc;
  // mini-batches of 17 .. 32 tokens: two tiles of token rows, at head_dim 32 only (the reference's own tile table,
  // rust/fused/src/linear_fused_tile/mod.rs:31-38, ends at (32, 32))
  if (d->mini_batch > 32 || (d->mini_batch > 16 && d->head_dim != 32))
    return fail(TTT_ERR_UNSUPPORTED, "mini_batch %d has no kernel at head_dim %d (up to 16; up to 32 at head_dim 32)",
                d->mini_batch, d->head_dim);
  if (d->head_dim != 32 && d->head_dim != 64 && d->head_dim != 96 && d->head_dim != 128)
    return fail(TTT_ERR_UNSUPPORTED, "TTT-Linear head_dim %d has no kernel (32, 64, 96, 128)", d->head_dim);
  return TTT_OK;
}

int64_t ttt_linear_num_checkpoints(const ttt_desc* d) {
  if (check_common(d) != TTT_OK) return -1;
  const int64_t n = d->seq / d->mini_batch;
  return (n + d->checkpoint_interval - 1) / d->checkpoint_interval;
}

}  // extern "C"

namespace {
// ttt_linear_fwd in two steps, so that a caller with several problems of one shape (ttt_stack_fwd) can check and
// describe each and launch them together: the argument block, then the launch of n of them.
int prepare_linear_fwd(const ttt_desc* d, const void* xq, const void* xk, const void* xv, const float* W0,
                       const float* b0, const float* token_eta, const void* lr, const float* gamma,
                       const float* beta, void* out, float* W_out, float* b_out, float* W_ckpt, float* b_ckpt,
                       ttt::LinearFwdArgs* pa) {
  int rc = ttt_linear_supported(d);
  if (rc != TTT_OK) return rc;
  if (!xq || !xk || !xv || !W0 || !b0 || !token_eta || !lr || !gamma || !beta || !out || !W_out || !b_out)
    return fail(TTT_ERR_NULL, "ttt_linear_fwd: a required pointer is NULL");
  if ((W_ckpt == nullptr) != (b_ckpt == nullptr))
    return fail(TTT_ERR_NULL, "W_ckpt and b_ckpt must both be given or both be NULL");
  if (!aligned16(xq) || !aligned16(xk) || !aligned16(xv) || !aligned16(out))
    return fail(TTT_ERR_SHAPE, "xq/xk/xv/out must be 16-byte aligned");
  ttt::LinearFwdArgs& a = *pa;
  a.xq = xq; a.xk = xk; a.xv = xv; a.W0 = W0; a.b0 = b0; a.token_eta = token_eta; a.lr = lr;
  a.gamma = gamma; a.beta = beta; a.out = out; a.W_out = W_out; a.b_out = b_out;
  a.W_ckpt = W_ckpt; a.b_ckpt = b_ckpt; a.xin = nullptr;
  a.B = d->batch; a.H = d->heads; a.seq = d->seq; a.K = d->mini_batch;
  a.seq_stride = d->seq_stride > 0 ? d->seq_stride : d->seq;
  a.n_stages = d->seq / d->mini_batch;
  a.ckpt_interval = d->checkpoint_interval;
  a.n_ckpt = (int)ttt_linear_num_checkpoints(d);
  a.state_per_batch = d->state_per_batch ? 1 : 0;
  if (W_ckpt != nullptr && d->checkpoint_format == TTT_CKPT_FACTORS) {
    rc = check_factors(d);
    if (rc != TTT_OK) return rc;
  }
  a.ckpt_packed = W_ckpt == nullptr ? 0
                  : ckpt_format_of(d) == TTT_CKPT_PACKED ? 1
                  : ckpt_format_of(d) == TTT_CKPT_FACTORS ? ttt::kCkptFactors : 0;
  a.eps = d->eps;
  // the LDS-tile forward exists for head_dim 96/128 only; elsewhere the hint names no kernel and is ignored
  const bool want_lds = (d->kernel_hint & TTT_HINT_LDS_TILES) != 0 && d->head_dim > 64;
  if (a.ckpt_packed == 1 && (d->checkpoint_interval != 1 || want_lds))
    return fail(TTT_ERR_UNSUPPORTED, "packed checkpoints need checkpoint_interval 1 and the register-resident kernels");
  if (d->mini_batch > 16 && a.ckpt_packed != 0)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_fwd: mini_batch %d > 16 writes f32 row-major checkpoints only", d->mini_batch);
  return TTT_OK;
}

int dispatch_linear_fwd_pack(const ttt_desc* d, const ttt::LinearFwdArgs* a, unsigned ny, hipStream_t s) {
  const bool want_lds = (d->kernel_hint & TTT_HINT_LDS_TILES) != 0 && d->head_dim > 64;
  const bool f32 = d->io_dtype == TTT_F32;
  if (d->mini_batch > 16)  // head_dim 32 (ttt_linear_supported): the LDS-tile kernel on two tiles of token rows
    return f32 ? launch_linear_fwd_lds<ttt::F32, 32, 2>(a, ny, s)
               : (d->kernel_hint & TTT_HINT_LDS_TILES) ? launch_linear_fwd_lds<ttt::BF16, 32, 2>(a, ny, s)
                                                       : launch_linear_fwd_lds<ttt::BF16, 32, 2, true>(a, ny, s);
  switch (d->head_dim) {
    case 32: return f32 ? launch_linear_fwd<ttt::F32, 32>(a, d->kernel_hint, ny, s) : launch_linear_fwd<ttt::BF16, 32>(a, d->kernel_hint, ny, s);
    case 64: return f32 ? launch_linear_fwd<ttt::F32, 64>(a, d->kernel_hint, ny, s) : launch_linear_fwd<ttt::BF16, 64>(a, d->kernel_hint, ny, s);
    default: break;
  }
  if (want_lds) {
    if (d->head_dim == 96)
      return f32 ? launch_linear_fwd_lds<ttt::F32, 96>(a, ny, s) : launch_linear_fwd_lds<ttt::BF16, 96>(a, ny, s);
    return f32 ? launch_linear_fwd_lds<ttt::F32, 128>(a, ny, s) : launch_linear_fwd_lds<ttt::BF16, 128>(a, ny, s);
  }
  if (d->head_dim == 96)
    return f32 ? launch_linear_fwd_wide<ttt::F32, 96>(a, ny, s) : launch_linear_fwd_wide<ttt::BF16, 96>(a, ny, s);
  return f32 ? launch_linear_fwd_wide<ttt::F32, 128>(a, ny, s) : launch_linear_fwd_wide<ttt::BF16, 128>(a, ny, s);
}

// n problems of one shape: kMaxProblems per launch
int dispatch_linear_fwd(const ttt_desc* d, const ttt::LinearFwdArgs* probs, int n, hipStream_t s) {
  for (int p = 0; p < n; p += ttt::kMaxProblems) {
    const int cnt = n - p < ttt::kMaxProblems ? n - p : ttt::kMaxProblems;
    const int rc = dispatch_linear_fwd_pack(d, probs + p, (unsigned)cnt, s);
    if (rc != TTT_OK) return rc;
  }
  return TTT_OK;
}
}  // namespace

namespace {
template <class T, int D, int NL>
int launch_mlpn(const ttt::MlpNFwdArgs& a, hipStream_t s) {
  constexpr auto kern = ttt::ttt_mlpn_fwd_kernel<T, D, NL>;
  constexpr size_t bytes = ttt::MlpNLds<D, NL>::BYTES;
  int rc = opt_in_lds<kern>(bytes);
  if (rc != TTT_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)(a.B * a.H)), dim3(512), bytes, s, a);
  return hip_status(hipGetLastError(), "ttt_mlpn_fwd launch");
}
}  // namespace

extern "C" {

int ttt_linear_fwd(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                   const float* W0, const float* b0, const float* token_eta, const void* lr,
                   const float* gamma, const float* beta, void* out, float* W_out, float* b_out,
                   float* W_ckpt, float* b_ckpt, void* stream) {
  ttt::LinearFwdArgs a;
  int rc = prepare_linear_fwd(d, xq, xk, xv, W0, b0, token_eta, lr, gamma, beta, out, W_out, b_out, W_ckpt, b_ckpt, &a);
  if (rc != TTT_OK) return rc;
  return dispatch_linear_fwd(d, &a, 1, static_cast<hipStream_t>(stream));
}

int ttt_mlpn_supported(const ttt_desc* d, int n_hidden) {
  int rc = check_common(d);
  if (rc != TTT_OK) return rc;
  if (d->mini_batch > 16) return fail(TTT_ERR_UNSUPPORTED, "mini_batch %d > 16 has no kernel", d->mini_batch);
  const bool ok = (d->head_dim == 32 && n_hidden >= 2 && n_hidden <= 4) || (d->head_dim == 64 && n_hidden == 2);
  if (!ok)
    return fail(TTT_ERR_UNSUPPORTED,
                "ttt_mlpn_fwd: head_dim 32 with 2, 3 or 4 hidden layers, head_dim 64 with 2 (got head_dim %d, %d hidden "
                "layers; one hidden layer is ttt_mlp_fwd)", d->head_dim, n_hidden);
  return TTT_OK;
}

int ttt_mlpn_fwd(const ttt_desc* d, int n_hidden, const void* xq, const void* xk, const void* xv,
                 const float* const* W0, const float* const* b0, const float* token_eta, const void* lr,
                 const float* gamma, const float* beta, void* out, float* const* W_out, float* const* b_out,
                 void* stream) {
  int rc = ttt_mlpn_supported(d, n_hidden);
  if (rc != TTT_OK) return rc;
  if (!xq || !xk || !xv || !W0 || !b0 || !token_eta || !lr || !gamma || !beta || !out || !W_out || !b_out)
    return fail(TTT_ERR_NULL, "ttt_mlpn_fwd: a required pointer is NULL");
  ttt::MlpNFwdArgs a;
  for (int i = 0; i < ttt::kMlpNMaxLayers; ++i) {
    a.W0[i] = a.b0[i] = nullptr;
    a.W[i] = a.b[i] = nullptr;
  }
  for (int i = 0; i <= n_hidden; ++i) {
    if (!W0[i] || !b0[i] || !W_out[i] || !b_out[i])
      return fail(TTT_ERR_NULL, "ttt_mlpn_fwd: layer %d: a required pointer is NULL", i);
    if (W_out[i] == W0[i])
      return fail(TTT_ERR_SHAPE, "ttt_mlpn_fwd: W_out[%d] is the live state and must not alias W0[%d]", i, i);
    a.W0[i] = W0[i]; a.b0[i] = b0[i]; a.W[i] = W_out[i]; a.b[i] = b_out[i];
  }
  a.xq = xq; a.xk = xk; a.xv = xv; a.token_eta = token_eta; a.lr = lr; a.gamma = gamma; a.beta = beta; a.out = out;
  a.B = d->batch; a.H = d->heads; a.seq = d->seq; a.K = d->mini_batch; a.n_stages = d->seq / d->mini_batch;
  a.seq_stride = d->seq_stride > 0 ? d->seq_stride : d->seq;
  a.state_per_batch = d->state_per_batch ? 1 : 0;
  a.eps = d->eps;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool f32 = d->io_dtype == TTT_F32;
  if (d->head_dim == 64) return f32 ? launch_mlpn<ttt::F32, 64, 2>(a, s) : launch_mlpn<ttt::BF16, 64, 2>(a, s);
  switch (n_hidden) {
    case 2: return f32 ? launch_mlpn<ttt::F32, 32, 2>(a, s) : launch_mlpn<ttt::BF16, 32, 2>(a, s);
    case 3: return f32 ? launch_mlpn<ttt::F32, 32, 3>(a, s) : launch_mlpn<ttt::BF16, 32, 3>(a, s);
    default: return f32 ? launch_mlpn<ttt::F32, 32, 4>(a, s) : launch_mlpn<ttt::BF16, 32, 4>(a, s);
  }
}

int ttt_linear_adam_supported(const ttt_desc* d) {
  int rc = ttt_linear_supported(d);
  if (rc != TTT_OK) return rc;
  if (d->mini_batch > 16) return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_adam_fwd: mini_batch up to 16 (got %d)", d->mini_batch);
  if (d->head_dim != 32 && d->head_dim != 64)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_adam_fwd: head_dim 32 or 64 (got %d)", d->head_dim);
  if ((d->kernel_hint & TTT_HINT_LDS_TILES) != 0)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_adam_fwd: the register-resident kernel only");
  return TTT_OK;
}

int ttt_linear_adam_fwd(const ttt_desc* d, const void* xq, const void* xk, const void* xv, const float* W0,
                        const float* b0, const float* Wm0, const float* bm0, const float* Wv0, const float* bv0,
                        int step0, float beta1, float beta2, float adam_eps, float adam_lr, const float* token_eta,
                        const void* lr, const float* gamma, const float* beta, void* out, float* W_out, float* b_out,
                        float* Wm_out, float* bm_out, float* Wv_out, float* bv_out, void* stream) {
  int rc = ttt_linear_adam_supported(d);
  if (rc != TTT_OK) return rc;
  const int n_in = (Wm0 != nullptr) + (bm0 != nullptr) + (Wv0 != nullptr) + (bv0 != nullptr);
  if (n_in != 0 && n_in != 4)
    return fail(TTT_ERR_NULL, "ttt_linear_adam_fwd: the four moments entering the call are given together or not at all");
  if (!Wm_out || !bm_out || !Wv_out || !bv_out)
    return fail(TTT_ERR_NULL, "ttt_linear_adam_fwd: a required pointer is NULL");
  if (step0 < 0 || (n_in == 0 && step0 != 0))
    return fail(TTT_ERR_SHAPE, "ttt_linear_adam_fwd: step0 must be >= 0, and 0 when no moments are given");
  if (!(beta1 >= 0.f && beta1 < 1.f) || !(beta2 >= 0.f && beta2 < 1.f) || !(adam_eps >= 0.f))
    return fail(TTT_ERR_SHAPE, "ttt_linear_adam_fwd: beta1, beta2 in [0, 1) and adam_eps >= 0");
  if (!aligned16(bm_out) || !aligned16(bv_out))
    return fail(TTT_ERR_SHAPE, "ttt_linear_adam_fwd: bm_out/bv_out must be 16-byte aligned");
  ttt::LinearFwdArgs a;
  rc = prepare_linear_fwd(d, xq, xk, xv, W0, b0, token_eta, lr, gamma, beta, out, W_out, b_out, nullptr, nullptr, &a);
  if (rc != TTT_OK) return rc;
  ttt::AdamArgs ad;
  ad.Wm0 = Wm0; ad.bm0 = bm0; ad.Wv0 = Wv0; ad.bv0 = bv0;
  ad.Wm_out = Wm_out; ad.bm_out = bm_out; ad.Wv_out = Wv_out; ad.bv_out = bv_out;
  ad.beta1 = beta1; ad.beta2 = beta2; ad.eps = adam_eps; ad.lr = adam_lr; ad.step0 = step0;
  const dim3 grid((unsigned)(a.B * a.H)), block(128);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool full = d->mini_batch == 16, f32 = d->io_dtype == TTT_F32;
  // head_dim 64 holds state and both moments in 96 registers per wave: the rows are prefetched one mini-batch ahead
  // there (two ahead would spill hundreds of registers), two ahead at head_dim 32
#define TTT_ADAM_LAUNCH(T_, D_, FULL_) \
  hipLaunchKernelGGL((ttt::ttt_linear_adam_fwd_kernel<T_, D_, 2, (D_ == 64 ? 1 : 2), FULL_>), grid, block, 0, s, a, ad)
  if (d->head_dim == 64) {
    if (f32) { if (full) TTT_ADAM_LAUNCH(ttt::F32, 64, true); else TTT_ADAM_LAUNCH(ttt::F32, 64, false); }
    else { if (full) TTT_ADAM_LAUNCH(ttt::BF16, 64, true); else TTT_ADAM_LAUNCH(ttt::BF16, 64, false); }
  } else {
    if (f32) { if (full) TTT_ADAM_LAUNCH(ttt::F32, 32, true); else TTT_ADAM_LAUNCH(ttt::F32, 32, false); }
    else { if (full) TTT_ADAM_LAUNCH(ttt::BF16, 32, true); else TTT_ADAM_LAUNCH(ttt::BF16, 32, false); }
  }
#undef TTT_ADAM_LAUNCH
  return hip_status(hipGetLastError(), "ttt_linear_adam_fwd launch");
}

int ttt_linear_fwd_fused_inputs_supported(const ttt_desc* d, int pos_wrap, int has_rope) {
  int rc = ttt_linear_supported(d);
  if (rc != TTT_OK) return rc;
  if (d->mini_batch > 16)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_fwd_fused_inputs: mini_batch up to 16 (got %d)", d->mini_batch);
  if (d->io_dtype != TTT_BF16 || (d->head_dim != 64 && d->head_dim != 32))
    return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_fwd_fused_inputs: bf16 I/O and head_dim 32 or 64 (got %s, %d)",
                d->io_dtype == TTT_BF16 ? "bf16" : "f32", d->head_dim);
  if (d->seq_stride != 0 && d->seq_stride != d->seq)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_fwd_fused_inputs: seq_stride must be 0");
  if (d->checkpoint_format == TTT_CKPT_FACTORS)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_fwd_fused_inputs: checkpoint formats f32 and packed only");
  if ((d->kernel_hint & TTT_HINT_LDS_TILES) != 0)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_linear_fwd_fused_inputs: the register-resident kernel only");
  if (has_rope && pos_wrap < 0) return fail(TTT_ERR_SHAPE, "pos_wrap must be >= 0");
  if (has_rope && pos_wrap > 0 && d->mini_batch % pos_wrap != 0)
    return fail(TTT_ERR_UNSUPPORTED,
                "ttt_linear_fwd_fused_inputs: pos_wrap %d must divide mini_batch %d (positions that repeat with the "
                "mini-batch) or be 0 (positions over the sequence)", pos_wrap, d->mini_batch);
  return TTT_OK;
}

int ttt_linear_fwd_fused_inputs(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                                const void* lr_logits, const float* lr_bias, float base_lr, const float* token_idx,
                                const float* learnable_token_idx, const float* rope_cos, const float* rope_sin,
                                int pos_offset, int pos_wrap, const float* W0, const float* b0, const float* gamma,
                                const float* beta, void* out, float* W_out, float* b_out, float* W_ckpt, float* b_ckpt,
                                void* xq_out, void* xk_out, void* xv_out, void* lr_out, float* token_eta_out,
                                void* stream) {
  if ((rope_cos == nullptr) != (rope_sin == nullptr))
    return fail(TTT_ERR_NULL, "rope_cos and rope_sin must both be given or both be NULL");
  int rc = ttt_linear_fwd_fused_inputs_supported(d, pos_wrap, rope_cos != nullptr);
  if (rc != TTT_OK) return rc;
  if (!lr_logits || !lr_bias || !token_idx || !learnable_token_idx)
    return fail(TTT_ERR_NULL, "ttt_linear_fwd_fused_inputs: a required pointer is NULL");
  if (pos_offset < 0) return fail(TTT_ERR_SHAPE, "pos_offset must be >= 0");
  if (!aligned16(xq_out) || !aligned16(xk_out) || !aligned16(xv_out))
    return fail(TTT_ERR_SHAPE, "xq_out/xk_out/xv_out must be 16-byte aligned");
  if ((rope_cos != nullptr && (reinterpret_cast<uintptr_t>(rope_cos) & 7u) != 0) ||
      (rope_sin != nullptr && (reinterpret_cast<uintptr_t>(rope_sin) & 7u) != 0))
    return fail(TTT_ERR_SHAPE, "rope_cos/rope_sin must be 8-byte aligned");
  ttt::LinearFwdArgs a;
  // the operand fields of the argument block are not read in this mode; the raw tensors stand in for the checks
  rc = prepare_linear_fwd(d, xq, xk, xv, W0, b0, token_idx, lr_logits, gamma, beta, out, W_out, b_out, W_ckpt, b_ckpt, &a);
  if (rc != TTT_OK) return rc;
  a.xq = a.xk = a.xv = a.lr = nullptr;
  a.token_eta = nullptr;
  a.seq_stride = d->seq;
  ttt::FusedInputsArgs fi;
  fi.xq = xq; fi.xk = xk; fi.xv = xv; fi.lr_logits = lr_logits; fi.lr_bias = lr_bias;
  fi.token_idx = token_idx; fi.learnable_token_idx = learnable_token_idx; fi.cos = rope_cos; fi.sin = rope_sin;
  fi.xq_out = xq_out; fi.xk_out = xk_out; fi.xv_out = xv_out; fi.lr_out = lr_out; fi.token_eta_out = token_eta_out;
  fi.lr_scale = base_lr / (float)d->head_dim;
  fi.pos_offset = pos_offset; fi.pos_wrap = pos_wrap;
  const bool per_token = rope_cos != nullptr && pos_wrap == 0;  // positions run over the sequence
  const bool full = d->mini_batch == 16;
  const dim3 grid((unsigned)(a.B * a.H)), block(128);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define TTT_FI_LAUNCH(D_, FULL_, RAW_) \
  hipLaunchKernelGGL((ttt::ttt_linear_fwd_fi_kernel<ttt::BF16, D_, 2, 2, FULL_, false, RAW_>), grid, block, 0, s, a, fi)
  if (d->head_dim == 64) {
    if (per_token) { if (full) TTT_FI_LAUNCH(64, true, 2); else TTT_FI_LAUNCH(64, false, 2); }
    else { if (full) TTT_FI_LAUNCH(64, true, 1); else TTT_FI_LAUNCH(64, false, 1); }
  } else {
    if (per_token) { if (full) TTT_FI_LAUNCH(32, true, 2); else TTT_FI_LAUNCH(32, false, 2); }
    else { if (full) TTT_FI_LAUNCH(32, true, 1); else TTT_FI_LAUNCH(32, false, 1); }
  }
#undef TTT_FI_LAUNCH
  return hip_status(hipGetLastError(), "ttt_linear_fwd_fused_inputs launch");
}

int ttt_linear_bwd_supported(const ttt_desc* d) {
  LinearBwdChoice ch;
  return choose_linear_bwd(d, &ch);
}

int ttt_linear_best_checkpoint_format(const ttt_desc* d) {
  int rc = ttt_linear_supported(d);
  if (rc != TTT_OK) return rc;
  // measured at head_dim 64 (125M shape): factors win up to 512 units, where the feature-split backward runs anyway;
  // beyond, the single-wave backward from packed states and the feature-split one from factors are even
  const bool factors_pay = d->seq / d->mini_batch >= 2 && (int64_t)d->batch * d->heads <= 512;
  // the first candidate, cheapest first, for which the backward has a kernel under this desc's interval and hint
  const int order[3] = {TTT_CKPT_FACTORS, TTT_CKPT_PACKED, TTT_CKPT_F32};
  for (int i = factors_pay ? 0 : 1; i < 3; ++i) {
    ttt_desc trial = *d;
    trial.checkpoint_format = order[i];
    LinearBwdChoice ch;
    rc = choose_linear_bwd(&trial, &ch);
    if (rc == TTT_OK) return order[i];
  }
  return rc;  // no format has a backward kernel: the status ttt_linear_bwd would return for the f32 format
}

}  // extern "C"

namespace {
// Whether a desc's TTT-Linear backward can spread every unit over two workgroups (producer and consumer,
// ttt_linear_bwd_pair_kernel): f32 I/O, whose reverse scan is bound by the f32 matrix instructions of the SIMDs that
// hold a unit, one checkpoint per mini-batch (row-major or packed), head_dim 32 or 64, at most 128 units.  A function
// of the desc alone, because the size of the workspace follows from it; the launch checks the device's CU count on top.
bool linear_bwd_pair_wanted(const ttt_desc* d) {
  LinearBwdChoice ch;
  if (choose_linear_bwd(d, &ch) != TTT_OK) return false;
  if (ch.kind != LinearBwdChoice::REG || d->io_dtype != TTT_F32) return false;
  if (d->head_dim != 32 && d->head_dim != 64) return false;
  if ((d->kernel_hint & (TTT_HINT_ONE_WORKGROUP | TTT_HINT_WAVES_MASK)) != 0) return false;
  if (d->seq / d->mini_batch < 2) return false;
  return (int64_t)d->batch * d->heads <= 128;
}
struct LinBwdPairWs {
  size_t hand, flags, total;
};
LinBwdPairWs linear_bwd_pair_ws(const ttt_desc* d) {
  const size_t U = (size_t)d->batch * d->heads;
  const size_t slot = d->head_dim == 64 ? ttt::LinBwdPair<64, true>::H_BYTES : ttt::LinBwdPair<32, true>::H_BYTES;
  static_assert(ttt::LinBwdPair<64, true>::H_BYTES == ttt::LinBwdPair<64, false>::H_BYTES, "one slot size per head_dim");
  LinBwdPairWs w;
  w.hand = 0;
  w.flags = U * ttt::kLinBwdPairSlots * slot;
  w.total = w.flags + U * ttt::kLinBwdPairFlagWords * sizeof(unsigned);
  return w;
}

int linear_bwd_impl(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                    const float* W0, const float* b0, const float* token_eta, const void* lr,
                    const float* gamma, const float* beta, const float* W_ckpt,
                    const float* b_ckpt, const void* d_out, const float* d_W_out,
                    const float* d_b_out, void* d_xq, void* d_xk, void* d_xv, float* d_W0,
                    float* d_b0, void* d_lr, float* d_token_eta, float* d_gamma, float* d_beta,
                    void* workspace, void* stream) {
  // the kernel is chosen (and a desc without one refused) before anything is enqueued
  LinearBwdChoice ch;
  int rc = choose_linear_bwd(d, &ch);
  if (rc != TTT_OK) return rc;
  bool pair = workspace != nullptr && linear_bwd_pair_wanted(d);
  if (pair) {
    if (!aligned16(workspace)) return fail(TTT_ERR_SHAPE, "ttt_linear_bwd_ws: workspace must be 16-byte aligned");
    int cus = 0;
    rc = device_cus(&cus);
    if (rc != TTT_OK) return rc;
    pair = 2 * (int64_t)d->batch * d->heads <= cus;  // every workgroup a CU of its own, both sides resident together
  }
  // W0/b0 are part of the saved state for interface parity; the state entering every stage is
  // rebuilt from the checkpoints (checkpoint 0 equals the initial state).
  (void)W0;
  (void)b0;
  if (!xq || !xk || !xv || !token_eta || !lr || !gamma || !beta || !d_out || !d_xq || !d_xk ||
      !d_xv || !d_W0 || !d_b0 || !d_lr || !d_token_eta || !d_gamma || !d_beta)
    return fail(TTT_ERR_NULL, "ttt_linear_bwd: a required pointer is NULL");
  if (!W_ckpt || !b_ckpt)
    return fail(TTT_ERR_NULL, "ttt_linear_bwd needs the W/b checkpoints written by ttt_linear_fwd");
  ttt::LinearBwdArgs a;
  a.xq = xq; a.xk = xk; a.xv = xv; a.token_eta = token_eta; a.lr = lr; a.gamma = gamma; a.beta = beta;
  a.W_ckpt = W_ckpt; a.b_ckpt = b_ckpt; a.d_out = d_out; a.d_W_out = d_W_out; a.d_b_out = d_b_out;
  a.d_xq = d_xq; a.d_xk = d_xk; a.d_xv = d_xv; a.d_W0 = d_W0; a.d_b0 = d_b0; a.d_lr = d_lr;
  a.d_token_eta = d_token_eta; a.d_gamma = d_gamma; a.d_beta = d_beta;
  a.B = d->batch; a.H = d->heads; a.seq = d->seq; a.K = d->mini_batch;
  a.seq_stride = d->seq_stride > 0 ? d->seq_stride : d->seq;
  a.n_stages = d->seq / d->mini_batch;
  a.ckpt_interval = d->checkpoint_interval;
  a.n_ckpt = (int)ttt_linear_num_checkpoints(d);
  a.ckpt_packed = ckpt_format_of(d) == TTT_CKPT_PACKED ? 1 : ckpt_format_of(d) == TTT_CKPT_FACTORS ? ttt::kCkptFactors : 0;
  a.eps = d->eps;
  const int D = d->head_dim;
  if (ch.kind != LinearBwdChoice::LDS &&
      (!aligned16(xq) || !aligned16(xk) || !aligned16(xv) || !aligned16(d_out) || !aligned16(d_xq) ||
       !aligned16(d_xk) || !aligned16(d_xv) || !aligned16(W_ckpt) || !aligned16(b_ckpt) ||
       ((size_t)a.seq_stride * D) % 8 != 0))
    return fail(TTT_ERR_SHAPE, "ttt_linear_bwd: tensors must be 16-byte aligned");
  if ((ch.w_global || ch.dw_global) && (!aligned16(W_ckpt) || !aligned16(d_W0)))
    return fail(TTT_ERR_SHAPE, "ttt_linear_bwd: W_ckpt and d_W0 must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // accumulated outputs start from zero; a fill kernel (not a memset node) so the sequence
  // can be captured into a graph
  const size_t hd = (size_t)d->heads * d->head_dim;
  {
    const size_t nmax = (size_t)d->seq > hd ? (size_t)d->seq : hd;
    hipLaunchKernelGGL(ttt::ttt_fill_zero3_kernel, dim3((unsigned)((nmax + 255) / 256)), dim3(256), 0, s, d_token_eta,
                       (size_t)d->seq, d_gamma, hd, d_beta, hd);
  }
  const unsigned grid = (unsigned)(a.B * a.H);
  const bool f32 = d->io_dtype == TTT_F32;
  const int waves = ch.waves;
  if (pair) {
    const LinBwdPairWs w = linear_bwd_pair_ws(d);
    ttt::LinearBwdPairArgs pa;
    pa.a = a;
    pa.hand = static_cast<unsigned char*>(workspace) + w.hand;
    pa.flags = reinterpret_cast<unsigned*>(static_cast<unsigned char*>(workspace) + w.flags);
    pa.spin_limit = (d->kernel_hint & TTT_HINT_TEST_LOST_PARTNER) ? 0u : (1u << 21);
    pa.agent_release = (d->kernel_hint & TTT_HINT_TEST_OTHER_XCD) ? 1 : 0;
    copy_or_zero(reinterpret_cast<float*>(pa.flags), nullptr, (size_t)grid * ttt::kLinBwdPairFlagWords, s);
    if (a.ckpt_packed)
      return D == 64 ? launch_linear_bwd_pair<64, true>(pa, s) : launch_linear_bwd_pair<32, true>(pa, s);
    return D == 64 ? launch_linear_bwd_pair<64, false>(pa, s) : launch_linear_bwd_pair<32, false>(pa, s);
  }
  if (ch.kind == LinearBwdChoice::LDS) {
    if (ch.w_global) return launch_linear_bwd<ttt::F32, 128, 1, true, true>(a, grid, s);
    // bf16 I/O: operands rounded to bf16 like the register-resident kernels, unless f32 products were asked for
    const bool bfops = !f32 && !(d->kernel_hint & TTT_HINT_LDS_TILES);
    if (ch.dw_global)
      return f32     ? launch_linear_bwd<ttt::F32, 96, 1, false, true>(a, grid, s)
             : bfops ? launch_linear_bwd<ttt::BF16, 96, 1, false, true, true>(a, grid, s)
                     : launch_linear_bwd<ttt::BF16, 96, 1, false, true>(a, grid, s);
    if (d->mini_batch > 16)
      return f32     ? launch_linear_bwd<ttt::F32, 32, 2>(a, grid, s)
             : bfops ? launch_linear_bwd<ttt::BF16, 32, 2, false, false, true>(a, grid, s)
                     : launch_linear_bwd<ttt::BF16, 32, 2>(a, grid, s);
    if (f32) return D == 64 ? launch_linear_bwd<ttt::F32, 64>(a, grid, s) : launch_linear_bwd<ttt::F32, 32>(a, grid, s);
    if (bfops)
      return D == 64 ? launch_linear_bwd<ttt::BF16, 64, 1, false, false, true>(a, grid, s)
                     : launch_linear_bwd<ttt::BF16, 32, 1, false, false, true>(a, grid, s);
    return D == 64 ? launch_linear_bwd<ttt::BF16, 64>(a, grid, s) : launch_linear_bwd<ttt::BF16, 32>(a, grid, s);
  }
  if (a.ckpt_packed == ttt::kCkptFactors) {
    if (D == 32) return launch_linear_bwd_mw<ttt::BF16, 32, 2, true, true>(a, grid, s);
    if (D == 64)
      return waves == 2 ? launch_linear_bwd_mw<ttt::BF16, 64, 2, true, true>(a, grid, s)
                        : launch_linear_bwd_mw<ttt::BF16, 64, 4, true, true>(a, grid, s);
    return launch_linear_bwd_mw<ttt::BF16, 96, 3, true, true>(a, grid, s);
  }
  if (f32 && a.ckpt_packed) {
    if (D == 32) return launch_linear_bwd_mw<ttt::F32, 32, 2, true>(a, grid, s);
    if (D == 64) return launch_linear_bwd_mw<ttt::F32, 64, 4, true>(a, grid, s);
    return launch_linear_bwd_mw<ttt::F32, 96, 3, true>(a, grid, s);
  }
  if (f32) {
    if (D == 32) return launch_linear_bwd_mw<ttt::F32, 32, 2>(a, grid, s);
    if (D == 64) return waves == 2 ? launch_linear_bwd_mw<ttt::F32, 64, 2>(a, grid, s)
                                   : launch_linear_bwd_mw<ttt::F32, 64, 4>(a, grid, s);
    return launch_linear_bwd_mw<ttt::F32, 96, 3>(a, grid, s);
  }
  if (a.ckpt_packed) {
    if (D == 32) return waves > 1 ? launch_linear_bwd_mw<ttt::BF16, 32, 2, true>(a, grid, s) : launch_linear_bwd_rr<32, true>(a, grid, s);
    if (D == 64) {
      if (waves == 2) return launch_linear_bwd_mw<ttt::BF16, 64, 2, true>(a, grid, s);
      return waves > 1 ? launch_linear_bwd_mw<ttt::BF16, 64, 4, true>(a, grid, s) : launch_linear_bwd_rr<64, true>(a, grid, s);
    }
    if (D == 96) return launch_linear_bwd_mw<ttt::BF16, 96, 3, true>(a, grid, s);
    return launch_linear_bwd_mw<ttt::BF16, 128, 4, true>(a, grid, s);
  }
  if (D == 32) return waves > 1 ? launch_linear_bwd_mw<ttt::BF16, 32, 2>(a, grid, s) : launch_linear_bwd_rr<32>(a, grid, s);
  if (D == 64) {
    if (waves == 1) return launch_linear_bwd_rr<64>(a, grid, s);
    return waves == 2 ? launch_linear_bwd_mw<ttt::BF16, 64, 2>(a, grid, s)
                      : launch_linear_bwd_mw<ttt::BF16, 64, 4>(a, grid, s);
  }
  if (D == 96) return launch_linear_bwd_mw<ttt::BF16, 96, 3>(a, grid, s);
  return launch_linear_bwd_mw<ttt::BF16, 128, 4>(a, grid, s);
}
}  // namespace

extern "C" {

int ttt_linear_bwd(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                   const float* W0, const float* b0, const float* token_eta, const void* lr,
                   const float* gamma, const float* beta, const float* W_ckpt,
                   const float* b_ckpt, const void* d_out, const float* d_W_out,
                   const float* d_b_out, void* d_xq, void* d_xk, void* d_xv, float* d_W0,
                   float* d_b0, void* d_lr, float* d_token_eta, float* d_gamma, float* d_beta,
                   void* stream) {
  return linear_bwd_impl(d, xq, xk, xv, W0, b0, token_eta, lr, gamma, beta, W_ckpt, b_ckpt, d_out, d_W_out, d_b_out,
                         d_xq, d_xk, d_xv, d_W0, d_b0, d_lr, d_token_eta, d_gamma, d_beta, nullptr, stream);
}

int64_t ttt_linear_bwd_workspace_bytes(const ttt_desc* d) {
  LinearBwdChoice ch;
  const int rc = choose_linear_bwd(d, &ch);
  if (rc != TTT_OK) return rc;
  return linear_bwd_pair_wanted(d) ? (int64_t)linear_bwd_pair_ws(d).total : 0;
}

int ttt_linear_bwd_ws(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                      const float* W0, const float* b0, const float* token_eta, const void* lr,
                      const float* gamma, const float* beta, const float* W_ckpt,
                      const float* b_ckpt, const void* d_out, const float* d_W_out,
                      const float* d_b_out, void* d_xq, void* d_xk, void* d_xv, float* d_W0,
                      float* d_b0, void* d_lr, float* d_token_eta, float* d_gamma, float* d_beta,
                      void* workspace, void* stream) {
  return linear_bwd_impl(d, xq, xk, xv, W0, b0, token_eta, lr, gamma, beta, W_ckpt, b_ckpt, d_out, d_W_out, d_b_out,
                         d_xq, d_xk, d_xv, d_W0, d_b0, d_lr, d_token_eta, d_gamma, d_beta, workspace, stream);
}

int ttt_mlp_supported(const ttt_desc* d) {
  int rc = check_common(d);
  if (rc != TTT_OK) return rc;
  if (d->mini_batch > 16)
    return fail(TTT_ERR_UNSUPPORTED, "mini_batch %d > 16 has no kernel", d->mini_batch);
  if (d->head_dim != 32 && d->head_dim != 64 && d->head_dim != 96 && d->head_dim != 128)
    return fail(TTT_ERR_UNSUPPORTED, "TTT-MLP head_dim %d has no kernel (32, 64, 96, 128)", d->head_dim);
  return TTT_OK;
}

}  // extern "C"

namespace {
// ttt_mlp_fwd in the same two steps as the Linear forward.
int prepare_mlp_fwd(const ttt_desc* d, const void* xq, const void* xk, const void* xv, const float* W1_0,
                    const float* b1_0, const float* W2_0, const float* b2_0, const float* token_eta, const void* lr,
                    const float* gamma, const float* beta, void* out, float* W1_out, float* b1_out, float* W2_out,
                    float* b2_out, ttt::MlpFwdArgs* pa) {
  int rc = ttt_mlp_supported(d);
  if (rc != TTT_OK) return rc;
  if (!xq || !xk || !xv || !W1_0 || !b1_0 || !W2_0 || !b2_0 || !token_eta || !lr || !gamma || !beta ||
      !out || !W1_out || !b1_out || !W2_out || !b2_out)
    return fail(TTT_ERR_NULL, "ttt_mlp_fwd: a required pointer is NULL");
  if (W1_out == W1_0 || W2_out == W2_0)
    return fail(TTT_ERR_SHAPE, "ttt_mlp_fwd: W1_out/W2_out are the live state and must not alias W1_0/W2_0");
  ttt::MlpFwdArgs& a = *pa;
  a.xq = xq; a.xk = xk; a.xv = xv; a.W1_0 = W1_0; a.b1_0 = b1_0; a.W2_0 = W2_0; a.b2_0 = b2_0;
  a.token_eta = token_eta; a.lr = lr; a.gamma = gamma; a.beta = beta; a.out = out;
  a.W1 = W1_out; a.b1 = b1_out; a.W2 = W2_out; a.b2 = b2_out;
  a.G1_save = nullptr; a.G2_save = nullptr; a.unit_base = 0; a.exchange_cleared = 0;
  a.spin_limit = (d->kernel_hint & TTT_HINT_TEST_LOST_PARTNER) ? 0 : (1 << 21);
  a.assume_other_xcd = (d->kernel_hint & TTT_HINT_TEST_OTHER_XCD) ? 1 : 0;
  a.B = d->batch; a.H = d->heads; a.seq = d->seq; a.K = d->mini_batch;
  a.seq_stride = d->seq_stride > 0 ? d->seq_stride : d->seq;
  a.n_stages = d->seq / d->mini_batch;
  a.state_per_batch = d->state_per_batch ? 1 : 0;
  a.eps = d->eps;
  return TTT_OK;
}

int dispatch_mlp_fwd_pack(const ttt_desc* d, const ttt::MlpFwdArgs* a, unsigned ny, hipStream_t s) {
  const bool f32 = d->io_dtype == TTT_F32;
  const bool want_lds = (d->kernel_hint & TTT_HINT_LDS_TILES) != 0;
  if (!f32 && d->head_dim <= 96 && !want_lds) {
    switch (d->head_dim) {
      case 32: return launch_mlp_fwd_rr<ttt::BF16, 32>(a, ny, s);
      case 64: return launch_mlp_fwd_rr<ttt::BF16, 64>(a, ny, s);
      default: return launch_mlp_fwd_rr<ttt::BF16, 96>(a, ny, s);
    }
  }
  switch (d->head_dim) {
    case 32: return f32 ? launch_mlp_fwd<ttt::F32, 32>(a, ny, s) : launch_mlp_fwd<ttt::BF16, 32>(a, ny, s);
    case 64: return f32 ? launch_mlp_fwd<ttt::F32, 64>(a, ny, s) : launch_mlp_fwd<ttt::BF16, 64>(a, ny, s);
    case 96: return f32 ? launch_mlp_fwd<ttt::F32, 96>(a, ny, s) : launch_mlp_fwd<ttt::BF16, 96>(a, ny, s);
    default: return f32 ? launch_mlp_fwd<ttt::F32, 128>(a, ny, s) : launch_mlp_fwd<ttt::BF16, 128>(a, ny, s);
  }
}

int dispatch_mlp_fwd(const ttt_desc* d, const ttt::MlpFwdArgs* probs, int n, hipStream_t s) {
  // bf16 I/O, d <= 96: the state fits the register file of one CU; d = 128: of two (see uses_two_cu_mlp).
  // TTT_HINT_LDS_TILES forces the LDS-tile kernel (f32 products, state in global memory) that the other cases use.
  bool two_cu = false;
  int rc = uses_two_cu_mlp(d, n, &two_cu);
  if (rc != TTT_OK) return rc;
  if (two_cu) return d->head_dim == 128 ? launch_mlp_fwd_cl2<128>(probs, n, s) : launch_mlp_fwd_cl2<96>(probs, n, s);
  for (int p = 0; p < n; p += ttt::kMaxProblems) {
    const int cnt = n - p < ttt::kMaxProblems ? n - p : ttt::kMaxProblems;
    rc = dispatch_mlp_fwd_pack(d, probs + p, (unsigned)cnt, s);
    if (rc != TTT_OK) return rc;
  }
  return TTT_OK;
}
}  // namespace

extern "C" {

int ttt_mlp_fwd(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                const float* token_eta, const void* lr, const float* gamma, const float* beta,
                void* out, float* W1_out, float* b1_out, float* W2_out, float* b2_out,
                void* stream) {
  ttt::MlpFwdArgs a;
  int rc = prepare_mlp_fwd(d, xq, xk, xv, W1_0, b1_0, W2_0, b2_0, token_eta, lr, gamma, beta, out, W1_out, b1_out,
                           W2_out, b2_out, &a);
  if (rc != TTT_OK) return rc;
  return dispatch_mlp_fwd(d, &a, 1, static_cast<hipStream_t>(stream));
}

int ttt_mlp_fwd_lost_workgroups(int64_t* count) {
  if (!count) return fail(TTT_ERR_NULL, "ttt_mlp_fwd_lost_workgroups: count is NULL");
  unsigned int v = 0;
  int rc = hip_status(hipMemcpyFromSymbol(&v, HIP_SYMBOL(ttt::g_mlp_fwd_lost_workgroups), sizeof(v), 0, hipMemcpyDeviceToHost),
                      "hipMemcpyFromSymbol(status word)");
  if (rc != TTT_OK) return rc;
  *count = (int64_t)v;
  return TTT_OK;
}

int64_t ttt_mlp_bwd_workspace_bytes(const ttt_desc* d) {
  if (ttt_mlp_supported(d) != TTT_OK) return -1;
  return (int64_t)(MlpBwdWs(d).total * sizeof(float));
}

int ttt_mlp_bwd(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                const float* token_eta, const void* lr, const float* gamma, const float* beta,
                const void* d_out, const float* d_W1_out, const float* d_b1_out,
                const float* d_W2_out, const float* d_b2_out, void* d_xq, void* d_xk, void* d_xv,
                float* d_W1, float* d_b1, float* d_W2, float* d_b2, void* d_lr, float* d_token_eta,
                float* d_gamma, float* d_beta, void* workspace, void* stream) {
  return mlp_bwd_impl(d, xq, xk, xv, W1_0, b1_0, W2_0, b2_0, token_eta, lr, gamma, beta, d_out, d_W1_out,
                      d_b1_out, d_W2_out, d_b2_out, d_xq, d_xk, d_xv, d_W1, d_b1, d_W2, d_b2, d_lr,
                      d_token_eta, d_gamma, d_beta, workspace, stream);
}

int ttt_mlp_fwd_saving_supported(const ttt_desc* d) {
  int rc = ttt_mlp_supported(d);
  if (rc != TTT_OK) return rc;
  bool two_cu = false;
  rc = uses_two_cu_mlp(d, 1, &two_cu);
  if (rc != TTT_OK) return rc;
  if (two_cu)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_mlp_fwd_saving: the forward on pairs of CUs saves nothing for the backward "
                                     "(head_dim %d); call ttt_mlp_fwd and ttt_mlp_bwd", d->head_dim);
  return TTT_OK;
}

int ttt_mlp_fwd_saving(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                       const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                       const float* token_eta, const void* lr, const float* gamma, const float* beta,
                       void* out, float* W1_out, float* b1_out, float* W2_out, float* b2_out, void* saved,
                       void* stream) {
  int rc = ttt_mlp_fwd_saving_supported(d);
  if (rc != TTT_OK) return rc;
  if (!saved) return fail(TTT_ERR_NULL, "ttt_mlp_fwd_saving: saved is NULL");
  if (!aligned16(saved)) return fail(TTT_ERR_SHAPE, "ttt_mlp_fwd_saving: saved must be 16-byte aligned");
  ttt::MlpFwdArgs a;
  rc = prepare_mlp_fwd(d, xq, xk, xv, W1_0, b1_0, W2_0, b2_0, token_eta, lr, gamma, beta, out, W1_out, b1_out, W2_out,
                       b2_out, &a);
  if (rc != TTT_OK) return rc;
  const MlpBwdWs w(d);
  float* ws = static_cast<float*>(saved);
  a.G1_save = ws + w.G1s;
  a.G2_save = ws + w.G2s;
  hipStream_t s = static_cast<hipStream_t>(stream);
  rc = dispatch_mlp_fwd_pack(d, &a, 1, s);
  if (rc != TTT_OK) return rc;
  // the reverse scan walks the state back in place: it gets a copy of the final state of its own
  const size_t U = (size_t)d->batch * d->heads, D = d->head_dim, M = 4 * D;
  copy_or_zero(ws + w.W1, W1_out, U * D * M, s);
  copy_or_zero(ws + w.b1, b1_out, U * M, s);
  copy_or_zero(ws + w.W2, W2_out, U * M * D, s);
  copy_or_zero(ws + w.b2, b2_out, U * D, s);
  return hip_status(hipGetLastError(), "ttt_mlp_fwd_saving copies");
}

int ttt_mlp_bwd_saved(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                      const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                      const float* token_eta, const void* lr, const float* gamma, const float* beta,
                      const void* d_out, const float* d_W1_out, const float* d_b1_out,
                      const float* d_W2_out, const float* d_b2_out, void* d_xq, void* d_xk, void* d_xv,
                      float* d_W1, float* d_b1, float* d_W2, float* d_b2, void* d_lr, float* d_token_eta,
                      float* d_gamma, float* d_beta, void* saved, void* stream) {
  int rc = ttt_mlp_fwd_saving_supported(d);
  if (rc != TTT_OK) return rc;
  return mlp_bwd_impl(d, xq, xk, xv, W1_0, b1_0, W2_0, b2_0, token_eta, lr, gamma, beta, d_out, d_W1_out,
                      d_b1_out, d_W2_out, d_b2_out, d_xq, d_xk, d_xv, d_W1, d_b1, d_W2, d_b2, d_lr,
                      d_token_eta, d_gamma, d_beta, saved, stream, /*sweep=*/false);
}

int ttt_mlp_bwd_static(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                       const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                       const float* token_eta, const void* lr, const float* gamma, const float* beta,
                       const void* d_out, const float* d_W1_out, const float* d_b1_out,
                       const float* d_W2_out, const float* d_b2_out, void* d_xq, void* d_xk, void* d_xv,
                       float* d_W1, float* d_b1, float* d_W2, float* d_b2, void* d_lr,
                       float* d_token_eta, float* d_gamma, float* d_beta, void* stream) {
  int rc = ttt_mlp_supported(d);
  if (rc != TTT_OK) return rc;
  const int64_t need = ttt_mlp_bwd_workspace_bytes(d);
  if (need < 0 || (uint64_t)need > kMlpBwdScratchBytes)
    return fail(TTT_ERR_SHAPE,
                "ttt_mlp_bwd_static: this shape needs %lld bytes of scratch, the built-in buffer holds %llu; "
                "use ttt_mlp_bwd with a caller-owned workspace",
                (long long)need, (unsigned long long)kMlpBwdScratchBytes);
  void* ws = nullptr;
  rc = mlp_bwd_scratch(&ws);
  if (rc != TTT_OK) return rc;
  return mlp_bwd_impl(d, xq, xk, xv, W1_0, b1_0, W2_0, b2_0, token_eta, lr, gamma, beta, d_out, d_W1_out,
                      d_b1_out, d_W2_out, d_b2_out, d_xq, d_xk, d_xv, d_W1, d_b1, d_W2, d_b2, d_lr,
                      d_token_eta, d_gamma, d_beta, ws, stream);
}

}  // extern "C"

namespace {
// How a ttt_stack_fwd call is laid out.  Windows (l, j) = layer l on tokens [j*chunk, (j+1)*chunk); window (l, j)
// needs (l-1, j) and (l, j-1), so the windows of a diagonal l + j = t are independent.
struct StackPlan {
  int chunks;                     // number of windows
  std::vector<int> tok0, len;     // first token and length of every window
  size_t tensor;                  // bytes of one [B,H,seq,d] activation tensor, rounded up to 256
  std::vector<size_t> state_off;  // byte offset of layer l's spare state copy (more than one window only)
  int n_lin, n_mlp;               // windows of the two kinds
  size_t total;
};
int plan_stack(const ttt_desc* d, int32_t n_layers, const ttt_stack_layer* layers, int32_t chunk_tokens, StackPlan* p) {
  int rc = check_common(d);
  if (rc != TTT_OK) return rc;
  if (n_layers <= 0) return fail(TTT_ERR_SHAPE, "ttt_stack_fwd: n_layers must be positive (got %d)", n_layers);
  if (!layers) return fail(TTT_ERR_NULL, "ttt_stack_fwd: layers is NULL");
  if (d->seq_stride != 0 && d->seq_stride != d->seq)
    return fail(TTT_ERR_SHAPE, "ttt_stack_fwd: sequence windows (seq_stride) are not supported");
  if (chunk_tokens < 0) return fail(TTT_ERR_SHAPE, "ttt_stack_fwd: negative chunk_tokens");
  const int chunk = chunk_tokens == 0 ? d->seq : chunk_tokens;
  if (chunk % d->mini_batch != 0 || d->seq % chunk != 0)
    return fail(TTT_ERR_SHAPE, "ttt_stack_fwd: chunk_tokens (%d) must be a multiple of mini_batch (%d) that divides seq (%d)",
                chunk, d->mini_batch, d->seq);
  p->n_lin = p->n_mlp = 0;
  for (int l = 0; l < n_layers; ++l) {
    if (layers[l].kind != TTT_LAYER_LINEAR && layers[l].kind != TTT_LAYER_MLP)
      return fail(TTT_ERR_UNSUPPORTED, "ttt_stack_fwd: layer %d has kind %d", l, layers[l].kind);
    rc = layers[l].kind == TTT_LAYER_LINEAR ? ttt_linear_supported(d) : ttt_mlp_supported(d);
    if (rc != TTT_OK) return rc;
    if (d->mini_batch > 16) return fail(TTT_ERR_UNSUPPORTED, "ttt_stack_fwd: mini_batch up to 16 (got %d)", d->mini_batch);
  }
  // Windows of `chunk` tokens.  (Splitting the first window so that the upper layers start sooner was measured
  // and did not pay: the two-CU TTT-MLP kernel at the top of the benchmark stack bounds the call, and more
  // windows cost it more launches.)
  p->tok0.clear();
  p->len.clear();
  for (int t0 = 0; t0 < d->seq; t0 += chunk) {
    p->tok0.push_back(t0);
    p->len.push_back(chunk);
  }
  p->chunks = (int)p->tok0.size();
  for (int l = 0; l < n_layers; ++l) (layers[l].kind == TTT_LAYER_LINEAR ? p->n_lin : p->n_mlp) += p->chunks;
  const size_t es = d->io_dtype == TTT_BF16 ? 2 : 4;
  const size_t D = d->head_dim, U = (size_t)d->batch * d->heads, M = 4 * D;
  auto up = [](size_t n) { return (n + 255) / 256 * 256; };
  p->tensor = up(U * d->seq * D * es);
  size_t off = 3 * p->tensor;
  p->state_off.assign(n_layers, 0);
  if (p->chunks > 1) {
    for (int l = 0; l < n_layers; ++l) {
      p->state_off[l] = off;
      const size_t floats = layers[l].kind == TTT_LAYER_MLP ? U * (2 * D * M + M + D) : U * (D * D + D);
      off += up(floats * sizeof(float));
    }
  }
  p->total = off;
  return TTT_OK;
}

}  // namespace

extern "C" {

int64_t ttt_stack_fwd_workspace_bytes(const ttt_desc* d, int32_t n_layers, const ttt_stack_layer* layers,
                                      int32_t chunk_tokens) {
  StackPlan p;
  if (plan_stack(d, n_layers, layers, chunk_tokens, &p) != TTT_OK) return -1;
  return (int64_t)p.total;
}

int ttt_stack_fwd(const ttt_desc* d, int32_t n_layers, const ttt_stack_layer* layers, const float* token_eta,
                  void* out, void* workspace, int32_t chunk_tokens, void* aux_stream, void* stream) {
  StackPlan p;
  int rc = plan_stack(d, n_layers, layers, chunk_tokens, &p);
  if (rc != TTT_OK) return rc;
  if (!token_eta || !out || !workspace) return fail(TTT_ERR_NULL, "ttt_stack_fwd: a required pointer is NULL");
  if (!aligned16(workspace) || !aligned16(out)) return fail(TTT_ERR_SHAPE, "ttt_stack_fwd: out and workspace must be 16-byte aligned");
  if (aux_stream != nullptr && aux_stream == stream)
    return fail(TTT_ERR_SHAPE, "ttt_stack_fwd: aux_stream must differ from stream");
  const size_t es = d->io_dtype == TTT_BF16 ? 2 : 4;
  const size_t D = d->head_dim, U = (size_t)d->batch * d->heads, seq = d->seq, M = 4 * D;
  const int C = p.chunks;
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  unsigned char* sums[3] = {ws, ws + p.tensor, ws + 2 * p.tensor};
  hipStream_t main_s = static_cast<hipStream_t>(stream);
  const bool two_lanes = aux_stream != nullptr && p.n_lin > 0 && p.n_mlp > 0;
  hipStream_t lane_s[2] = {main_s, two_lanes ? static_cast<hipStream_t>(aux_stream) : main_s};

  // ---- pass 1: check and describe every window; nothing is enqueued before all of them are accepted
  // A group = the windows of one kind on one diagonal.  before / after: input sums launched ahead of the group's
  // kernels (for its own windows) and behind them (for windows of the other kind on the next diagonal whose layer
  // below is in this group: formed on the producer's stream, they are off the consumer's).
  struct Group {
    int t, kind, first, count;
    bool waits_other;
    std::vector<ttt::LayerInputsArgs> before, after;
  };
  std::vector<ttt::LinearFwdArgs> lin;
  std::vector<ttt::MlpFwdArgs> mlp;
  std::vector<int> mlp_first;  // the first windows of the TTT-MLP layers (indices into mlp)
  std::vector<Group> groups;
  for (int l = 0; l < n_layers; ++l) {
    const ttt_stack_layer& L = layers[l];
    if (!L.pq || !L.pk || !L.pv) return fail(TTT_ERR_NULL, "ttt_stack_fwd: layer %d: a required pointer is NULL", l);
    if (!aligned16(L.pq) || !aligned16(L.pk) || !aligned16(L.pv))
      return fail(TTT_ERR_SHAPE, "ttt_stack_fwd: layer %d: pq/pk/pv must be 16-byte aligned", l);
  }
  // bf16 I/O at head_dim 64 and 128: the TTT-Linear kernels form x + pq, x + pk, x + pv in their own loads (in place:
  // x is what the layer below left in `out`), so those windows need no launch and no workspace for their input sums
  const bool fuse_linear_sums = d->io_dtype == TTT_BF16 && (d->head_dim == 64 || d->head_dim == 128) &&
                                (d->kernel_hint & (TTT_HINT_LDS_TILES | TTT_HINT_WAVES_MASK)) == 0;
  for (int t = 0; t < C + n_layers - 1; ++t) {
    for (int kind = 0; kind < 2; ++kind) {
      Group g{t, kind, kind == TTT_LAYER_LINEAR ? (int)lin.size() : (int)mlp.size(), 0, false, {}, {}};
      for (int l = 0; l < n_layers; ++l) {
        const int j = t - l;
        const ttt_stack_layer& L = layers[l];
        if (j < 0 || j >= C || L.kind != kind) continue;
        const bool is_mlp = kind == TTT_LAYER_MLP;
        const size_t tok0 = (size_t)p.tok0[j];
        const size_t woff = tok0 * D * es;  // byte offset of the window inside a unit's rows
        const unsigned char *q = static_cast<const unsigned char*>(L.pq) + woff, *k = static_cast<const unsigned char*>(L.pk) + woff,
                            *v = static_cast<const unsigned char*>(L.pv) + woff;
        unsigned char* ow = static_cast<unsigned char*>(out) + woff;  // `out` is the hand-over tensor too
        const void* x_in = nullptr;
        if (l > 0 && !is_mlp && fuse_linear_sums) {
          // the TTT-Linear kernel forms x + projections itself, reading x from `out` in place
          x_in = ow;
          if (layers[l - 1].kind != kind) g.waits_other = true;
        } else if (l > 0) {
          // window j of the sums tensors is free: its previous user (l-1, j) is done before this window starts
          ttt::LayerInputsArgs a;
          a.x = ow; a.pq = q; a.pk = k; a.pv = v;
          a.xq = sums[0] + woff; a.xk = sums[1] + woff; a.xv = sums[2] + woff;
          a.win16 = (size_t)p.len[j] * D * es / 16;
          a.pitch16 = seq * D * es / 16;
          a.n16 = U * a.win16;
          q = sums[0] + woff; k = sums[1] + woff; v = sums[2] + woff;
          if (layers[l - 1].kind != kind) {
            g.waits_other = true;
            // the producer's group: the other kind on the previous diagonal (it holds window (l-1, j), so it exists
            // and is one of the last two groups pushed)
            Group* prod = nullptr;
            for (size_t i = groups.size(); i-- > 0 && groups[i].t >= t - 1;)
              if (groups[i].t == t - 1 && groups[i].kind != kind) prod = &groups[i];
            if (prod == nullptr) return fail(TTT_ERR_SHAPE, "ttt_stack_fwd: internal: no group for window (%d, %d)", l - 1, j);
            (two_lanes ? prod->after : g.before).push_back(a);
          } else {
            g.before.push_back(a);
          }
        }
        ttt_desc ld = *d;
        ld.seq = p.len[j];
        ld.seq_stride = C > 1 ? d->seq : 0;
        ld.checkpoint_interval = 1;
        ld.checkpoint_format = TTT_CKPT_F32;
        // state: window 0 starts from the layer's parameters; window j writes the caller's buffers when the
        // number of windows still to come is even, the spare copy otherwise; window j + 1 reads what j wrote
        float* spare = C > 1 ? reinterpret_cast<float*>(ws + p.state_off[l]) : nullptr;
        float* sp[4] = {spare, nullptr, nullptr, nullptr};
        if (spare) {
          sp[1] = is_mlp ? spare + U * D * M : spare + U * D * D;
          if (is_mlp) {
            sp[2] = sp[1] + U * M;
            sp[3] = sp[2] + U * M * D;
          }
        }
        float* user[4] = {L.W1_out, L.b1_out, L.W2_out, L.b2_out};
        float* const* to = ((C - 1 - j) % 2 == 0) ? user : sp;
        float* const* from = ((C - j) % 2 == 0) ? user : sp;
        const float *W1i = L.W1, *b1i = L.b1, *W2i = L.W2, *b2i = L.b2;
        if (j > 0) {
          ld.state_per_batch = 1;
          W1i = from[0]; b1i = from[1]; W2i = from[2]; b2i = from[3];
        }
        const unsigned char* lr = L.lr ? static_cast<const unsigned char*>(L.lr) + tok0 * es : nullptr;
        if (!is_mlp) {
          ttt::LinearFwdArgs a;
          rc = prepare_linear_fwd(&ld, q, k, v, W1i, b1i, token_eta, lr, L.gamma, L.beta, ow, to[0], to[1], nullptr, nullptr, &a);
          if (rc != TTT_OK) return rc;
          a.xin = x_in;
          lin.push_back(a);
        } else {
          ttt::MlpFwdArgs a;
          rc = prepare_mlp_fwd(&ld, q, k, v, W1i, b1i, W2i, b2i, token_eta, lr, L.gamma, L.beta, ow, to[0], to[1], to[2], to[3], &a);
          if (rc != TTT_OK) return rc;
          if (j == 0) mlp_first.push_back((int)mlp.size());
          mlp.push_back(a);
        }
        ++g.count;
      }
      if (g.count > 0) groups.push_back(g);
    }
  }

  // ---- pass 2: the launches, diagonal by diagonal
  // events (two lanes only): created here and destroyed before returning; the runtime keeps a recorded event
  // alive until the work it marks has finished
  std::vector<hipEvent_t> ev;
  bool forked = false;  // the second stream has been made to wait for `stream` and has not been joined back yet
  auto cleanup = [&](int r) {
    if (forked) {
      // an error between fork and join: `stream` still has to wait for whatever the second stream was given, or a
      // caller that is capturing `stream` into a graph is left with a branch that never rejoins (an invalid
      // capture), and any caller with work on the second stream that nothing orders.  Best effort: the call is
      // failing already and reports its first error.
      hipEvent_t e = nullptr;
      if (hipEventCreateWithFlags(&e, hipEventDisableTiming) == hipSuccess) {
        ev.push_back(e);
        if (hipEventRecord(e, lane_s[1]) == hipSuccess) (void)hipStreamWaitEvent(main_s, e, 0);
      }
      forked = false;
    }
    for (hipEvent_t e : ev) (void)hipEventDestroy(e);
    return r;
  };
  auto mark = [&](hipStream_t s, hipEvent_t* e) {
    int r = hip_status(hipEventCreateWithFlags(e, hipEventDisableTiming), "hipEventCreateWithFlags");
    if (r != TTT_OK) return r;
    ev.push_back(*e);
    return hip_status(hipEventRecord(*e, s), "hipEventRecord");
  };
  auto wait = [&](hipStream_t s, hipEvent_t e) { return hip_status(hipStreamWaitEvent(s, e, 0), "hipStreamWaitEvent"); };
  if (two_lanes) {
    hipEvent_t fork;
    if ((rc = mark(main_s, &fork)) != TTT_OK) return cleanup(rc);
    if ((rc = wait(lane_s[1], fork)) != TTT_OK) return cleanup(rc);
    forked = true;
  }
  // The two-CU TTT-MLP kernel exchanges through the window's W2 output buffer, which has to be zero when it starts.
  // Nothing reads or writes that buffer before a layer's FIRST window, so those are cleared here, while the stream
  // of the TTT-MLP launches has nothing else to do, instead of in front of the kernel, where the fill competes with
  // the other stream's traffic on the path to the first TTT-MLP launch (88 us in the trace instead of 7).
  if (d->io_dtype != TTT_F32 && d->head_dim == 128 && (d->kernel_hint & TTT_HINT_LDS_TILES) == 0) {
    const size_t nz = U * 128 * 512;
    for (int i : mlp_first) {
      hipLaunchKernelGGL(ttt::ttt_fill_zero_kernel, dim3((unsigned)((nz + 255) / 256)), dim3(256), 0, lane_s[1], mlp[i].W2, nz);
      mlp[i].exchange_cleared = 1;
    }
  }
  auto input_sums = [&](const std::vector<ttt::LayerInputsArgs>& v, hipStream_t s) {
    for (size_t i = 0; i < v.size(); i += ttt::kMaxProblems) {
      const unsigned cnt = (unsigned)(v.size() - i < (size_t)ttt::kMaxProblems ? v.size() - i : (size_t)ttt::kMaxProblems);
      const ttt::LayerInputsArgs* a = &v[i];
      size_t n16 = 0;  // the grid covers the longest window, threads past the end of a shorter one exit
      for (unsigned k = 0; k < cnt; ++k) n16 = a[k].n16 > n16 ? a[k].n16 : n16;
      const dim3 grid((unsigned)((n16 + 255) / 256), cnt);
      if (d->io_dtype == TTT_F32)
        hipLaunchKernelGGL(ttt::ttt_layer_inputs_kernel<ttt::F32>, grid, dim3(256), 0, s, pack_of(a, cnt));
      else
        hipLaunchKernelGGL(ttt::ttt_layer_inputs_kernel<ttt::BF16>, grid, dim3(256), 0, s, pack_of(a, cnt));
    }
    return hip_status(hipGetLastError(), "ttt_stack_fwd (layer inputs) launch");
  };
  // done[kind][t & 1]: event after the lane's launches of diagonal t (done_t: which diagonal the slot holds)
  hipEvent_t done[2][2] = {{nullptr, nullptr}, {nullptr, nullptr}};
  int done_t[2][2] = {{-2, -2}, {-2, -2}};
  for (const Group& g : groups) {
    hipStream_t s = lane_s[g.kind];
    const int other = 1 - g.kind;
    // a window whose layer below is of the other kind waits for that lane's launches of the previous diagonal
    // (the lane's later work is in stream order behind them, so its latest event would do as well, but would wait
    // for more than is needed)
    if (two_lanes && g.waits_other) {
      const int slot = (g.t - 1) & 1;
      if (done_t[other][slot] != g.t - 1) return cleanup(fail(TTT_ERR_SHAPE, "ttt_stack_fwd: internal: missing event of diagonal %d", g.t - 1));
      if ((rc = wait(s, done[other][slot])) != TTT_OK) return cleanup(rc);
    }
    if ((rc = input_sums(g.before, s)) != TTT_OK) return cleanup(rc);
    ttt_desc ld = *d;  // only what chooses the kernel is read from it; the windows' lengths are in the argument blocks
    ld.seq = d->mini_batch;
    if (g.kind == TTT_LAYER_LINEAR)
      rc = dispatch_linear_fwd(&ld, &lin[g.first], g.count, s);
    else
      rc = dispatch_mlp_fwd(&ld, &mlp[g.first], g.count, s);
    if (rc != TTT_OK) return cleanup(rc);
    if ((rc = input_sums(g.after, s)) != TTT_OK) return cleanup(rc);
    if (two_lanes) {
      if ((rc = mark(s, &done[g.kind][g.t & 1])) != TTT_OK) return cleanup(rc);
      done_t[g.kind][g.t & 1] = g.t;
    }
  }
  if (two_lanes) {
    hipEvent_t join;
    if ((rc = mark(lane_s[1], &join)) != TTT_OK) return cleanup(rc);
    if ((rc = wait(main_s, join)) != TTT_OK) return cleanup(rc);
    forked = false;
  }
  return cleanup(TTT_OK);
}

int ttt_selftest_mfma_mixed(int order, int gap, float* out, void* stream) {
  if (!out) return fail(TTT_ERR_NULL, "ttt_selftest_mfma_mixed: out is NULL");
  if (order < 0 || order > 3 || (gap != 0 && gap != 4 && gap != 5))
    return fail(TTT_ERR_SHAPE, "ttt_selftest_mfma_mixed: order must be 0 .. 3 and gap 0, 4 or 5 (got %d, %d)", order, gap);
  hipLaunchKernelGGL(ttt::ttt_selftest_mfma_mixed_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), order, gap, out);
  return hip_status(hipGetLastError(), "ttt_selftest_mfma_mixed launch");
}

int ttt_inner_inputs(const ttt_desc* d, const void* xq, const void* xk, const void* xv,
                     const void* lr_logits, const float* lr_bias, float base_lr, const float* token_idx,
                     const float* learnable_token_idx, const float* rope_cos, const float* rope_sin,
                     int pos_offset, int pos_wrap, void* xq_out, void* xk_out, void* xv_out, void* lr_out,
                     float* token_eta_out, void* stream) {
  if (!d) return fail(TTT_ERR_NULL, "ttt_inner_inputs: desc is NULL");
  if (d->batch <= 0 || d->heads <= 0 || d->seq <= 0 || d->head_dim <= 0 || d->mini_batch <= 0)
    return fail(TTT_ERR_SHAPE, "ttt_inner_inputs: batch, heads, seq, head_dim, mini_batch must be positive");
  if (d->head_dim % 8 != 0)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_inner_inputs: head_dim %d is not a multiple of 8", d->head_dim);
  if (d->io_dtype != TTT_F32 && d->io_dtype != TTT_BF16)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_inner_inputs: io_dtype %d", d->io_dtype);
  if (!xq || !xk || !xv || !lr_logits || !lr_bias || !token_idx || !learnable_token_idx || !xq_out ||
      !xk_out || !xv_out || !lr_out || !token_eta_out)
    return fail(TTT_ERR_NULL, "ttt_inner_inputs: a required pointer is NULL");
  if ((rope_cos == nullptr) != (rope_sin == nullptr))
    return fail(TTT_ERR_NULL, "ttt_inner_inputs: rope_cos and rope_sin must both be given or both be NULL");
  if (pos_offset < 0 || pos_wrap < 0) return fail(TTT_ERR_SHAPE, "ttt_inner_inputs: negative position");
  if (!aligned16(xq) || !aligned16(xk) || !aligned16(xv) || !aligned16(xq_out) || !aligned16(xk_out) ||
      !aligned16(xv_out) || !aligned16(rope_cos) || !aligned16(rope_sin))
    return fail(TTT_ERR_SHAPE, "ttt_inner_inputs: activation and table pointers must be 16-byte aligned");
  ttt::InnerInputsArgs a;
  a.xq = xq; a.xk = xk; a.xv = xv; a.lr_logits = lr_logits; a.lr_bias = lr_bias; a.token_idx = token_idx;
  a.learnable_token_idx = learnable_token_idx; a.cos = rope_cos; a.sin = rope_sin;
  a.xq_out = xq_out; a.xk_out = xk_out; a.xv_out = xv_out; a.lr_out = lr_out; a.token_eta_out = token_eta_out;
  a.lr_scale = base_lr / (float)d->head_dim;
  a.B = d->batch; a.H = d->heads; a.seq = d->seq; a.D = d->head_dim; a.K = d->mini_batch;
  a.pos_offset = pos_offset; a.pos_wrap = pos_wrap;
  const size_t total = (size_t)a.B * a.seq * a.H * (a.D / 8);
  const dim3 grid((unsigned)((total + 255) / 256));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (d->io_dtype == TTT_F32)
    hipLaunchKernelGGL(ttt::ttt_inner_inputs_kernel<ttt::F32>, grid, dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL(ttt::ttt_inner_inputs_kernel<ttt::BF16>, grid, dim3(256), 0, s, a);
  return hip_status(hipGetLastError(), "ttt_inner_inputs launch");
}

int ttt_layer_epilogue(const ttt_desc* d, const void* inner_out, const float* post_norm_weight,
                       const float* post_norm_bias, float eps, const void* gate, void* out, void* stream) {
  if (!d) return fail(TTT_ERR_NULL, "ttt_layer_epilogue: desc is NULL");
  if (d->batch <= 0 || d->heads <= 0 || d->seq <= 0 || d->head_dim <= 0)
    return fail(TTT_ERR_SHAPE, "ttt_layer_epilogue: batch, heads, seq, head_dim must be positive");
  const int hidden = d->heads * d->head_dim;
  if (d->head_dim % 8 != 0 || hidden > 2048)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_layer_epilogue: head_dim %d (multiple of 8) / hidden %d (<= 2048)",
                d->head_dim, hidden);
  if (d->io_dtype != TTT_F32 && d->io_dtype != TTT_BF16)
    return fail(TTT_ERR_UNSUPPORTED, "ttt_layer_epilogue: io_dtype %d", d->io_dtype);
  if (!inner_out || !post_norm_weight || !post_norm_bias || !out)
    return fail(TTT_ERR_NULL, "ttt_layer_epilogue: a required pointer is NULL");
  if (!aligned16(inner_out) || !aligned16(out) || !aligned16(gate) || !aligned16(post_norm_weight) ||
      !aligned16(post_norm_bias))
    return fail(TTT_ERR_SHAPE, "ttt_layer_epilogue: pointers must be 16-byte aligned");
  ttt::LayerEpilogueArgs a;
  a.inner_out = inner_out; a.gamma = post_norm_weight; a.beta = post_norm_bias; a.gate = gate; a.out = out;
  a.B = d->batch; a.H = d->heads; a.seq = d->seq; a.D = d->head_dim; a.eps = eps;
  const int nch = hidden / 8, nc = nch <= 64 ? 1 : nch <= 128 ? 2 : 4;
  const dim3 grid((unsigned)(((size_t)a.B * a.seq + 3) / 4));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (d->io_dtype == TTT_F32)
    launch_epilogue<ttt::F32>(a, nc, grid, s);
  else
    launch_epilogue<ttt::BF16>(a, nc, grid, s);
  return hip_status(hipGetLastError(), "ttt_layer_epilogue launch");
}

}  // extern "C"
