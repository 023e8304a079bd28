// CASTLE cached decode step for gfx950: one streaming pass over the cache.
//
// Reference semantics: lookahead_keys_attention.py:166-203.  For every cached row k < t
//     a_k  = sigmoid(s qu_k . ku_t)            U_k <- U_k + a_k vu_t      (in place)
//     x_k  = s qc_t . kc_k - silu(s qc_t . U_k)
// and for the appended row t:  U_t = 0,  x_t = s qc_t . kc_t;  out = softmax(x) V.
// The pass is bandwidth bound: each cached element of qu, U, kc, vc is read once and U is
// written once (5 * t * d elements per head and step).  The t rows of one (b, h) are split
// over `splits` workgroups that each keep an online-softmax partial (acc, m, l) in fp32;
// decode_finish_kernel merges the partials, folds in row t and appends the new rows.
#include "castle_tiles.h"
#include "castle_params.h"
#include "castle_profile.h"
#include <mutex>

#ifndef CASTLE_DEC_PF
#define CASTLE_DEC_PF 1   // iterations of row pieces requested ahead in the stream kernel
#endif
#ifndef CASTLE_DEC_WGS
#define CASTLE_DEC_WGS 640   // workgroups the stream kernel aims for
#endif

namespace castle {

template <typename T> __device__ __forceinline__ T* view_row(const View4& v, int b, int h, int64_t row) {
  return reinterpret_cast<T*>(v.ptr) + (int64_t)b * v.sb + (int64_t)h * v.sh + row * v.sl;
}

template <typename T, int N> __device__ __forceinline__ void load_f32(const T* p, float (&dst)[N]) {
  typedef vec<T, N> vt;
  vt x = *reinterpret_cast<const vt*>(p);
#pragma unroll
  for (int e = 0; e < N; ++e) dst[e] = (float)x[e];
}

// One 16-byte piece of a U row to fp32 and back.  UH: the buffer is in the half-precision cache
// format (fp16 bits of U * kUHalfScale, saturated) whatever the element type T of the cache is.
template <typename T, int N, bool UH> __device__ __forceinline__ void u_unpack(vec<T, N> raw, float (&dst)[N]) {
  if constexpr (UH) {
    static_assert(sizeof(T) == 2, "the half-precision format replaces a 16-bit element type");
    const vec<fp16_t, N> x = __builtin_bit_cast(vec<fp16_t, N>, raw);
#pragma unroll
    for (int e = 0; e < N; ++e) dst[e] = (float)x[e] * kUHalfUnscale;
  } else {
#pragma unroll
    for (int e = 0; e < N; ++e) dst[e] = (float)raw[e];
  }
}
template <typename T, int N, bool UH> __device__ __forceinline__ vec<T, N> u_pack(const float (&src)[N]) {
  if constexpr (UH) {
    vec<fp16_t, N> x;
#pragma unroll
    for (int e = 0; e < N; ++e) x[e] = (fp16_t)__builtin_amdgcn_fmed3f(src[e] * kUHalfScale, -kHalfMax, kHalfMax);
    return __builtin_bit_cast(vec<T, N>, x);
  } else {
    vec<T, N> x;
#pragma unroll
    for (int e = 0; e < N; ++e) x[e] = (T)src[e];
    return x;
  }
}

template <int LPR> __device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int o = 1; o < LPR; o <<= 1) v += __shfl_xor(v, o);
  return v;
}

// One workgroup = 4 waves; a group of LPR = d / V lanes owns one cache row per iteration.
template <typename T, int HD, bool UH>
__global__ __launch_bounds__(kThreads) void decode_stream_kernel(DecodeArgs a) {
  constexpr int V = elem_traits<T>::vec16;   // elements per 16-byte lane load
  constexpr int LPR = HD / V;                // lanes per row
  constexpr int RPI = kThreads / LPR;        // rows per workgroup iteration
  typedef vec<T, V> vt;
  __shared__ float s_acc[kThreads / LPR][HD + 2];

  const int split = blockIdx.x, bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  int t = a.t_dev != nullptr ? *a.t_dev : a.t;
  if (t < 0 || t >= a.capacity) t = 0;   // out of range (device-side count only): no rows, the finish kernel writes nothing
  const int tid = threadIdx.x;
  const int grp = tid / LPR, sub = tid % LPR;
  const float c0 = a.scale, c1 = a.scale * kLog2e;

  // rows of this workgroup: [r0, r1), whole iterations of RPI rows
  const int per = ((t + a.splits - 1) / a.splits + RPI - 1) / RPI * RPI;
  const int r0 = split * per;
  const int r1 = min(t, r0 + per);

  float ku[V], vu[V], qc[V];
  load_f32<T, V>(view_row<T>(a.ku, b, h, 0) + sub * V, ku);
  load_f32<T, V>(view_row<T>(a.vu, b, h, 0) + sub * V, vu);
  load_f32<T, V>(view_row<T>(a.qc, b, h, 0) + sub * V, qc);
  if (a.rotary) {   // the new token sits at position t
#pragma unroll
    for (int e = 0; e < V / 2; ++e) {
      const int pair = sub * (V / 2) + e;
      CASTLE_ROPE_PAIR(ku[2 * e], ku[2 * e + 1], (float)t, pair, HD, false);
      CASTLE_ROPE_PAIR(vu[2 * e], vu[2 * e + 1], (float)t, pair, HD, false);
      CASTLE_ROPE_PAIR(qc[2 * e], qc[2 * e + 1], (float)t, pair, HD, false);
    }
  }

  // deferred write-back: the pending tokens' vu pieces of this lane, and whether this step writes U
  const bool deferred = a.pend_vu.ptr != nullptr;
  const int base0 = a.base0_dev != nullptr ? *a.base0_dev : a.base0;
  const int pbase = deferred ? decode_base(base0, t) : t;
  const int np = t - pbase;                                        // 0 .. kDecodeDefer - 1
  const bool write_u = !deferred || (t + 1) % kDecodeDefer == 0;
  float pv[kDecodeDefer][V];   // indexed by ring slot; zero where no pending token sits
#pragma unroll
  for (int sl = 0; sl < kDecodeDefer; ++sl) {
#pragma unroll
    for (int e = 0; e < V; ++e) pv[sl][e] = 0.f;
    const int j = pbase + ((sl - pbase % kDecodeDefer + kDecodeDefer) % kDecodeDefer);   // the token that would sit in this slot
    if (deferred && j < t) load_f32<T, V>(view_row<T>(a.pend_vu, b, h, sl) + sub * V, pv[sl]);
  }
  const int slot_t = t % kDecodeDefer;

  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = 0.f;
  float m = -INFINITY, l = 0.f;

  // The row pieces of the next PF iterations are requested before the current one is processed:
  // PF + 1 times the bytes in flight per wave, which is what a latency-bound streaming loop is short of.
  constexpr int PF = CASTLE_DEC_PF;
  vt nq[PF], nu[PF], nk[PF], nv[PF];
  vec<float, 4> ng[PF];
#pragma unroll
  for (int p = 0; p < PF; ++p) ng[p] = vec<float, 4>{0.f, 0.f, 0.f, 0.f};
  float* const gbase = deferred ? reinterpret_cast<float*>(a.pend_gate.ptr) + (int64_t)b * a.pend_gate.sb + (int64_t)h * a.pend_gate.sh : nullptr;
  auto request = [&](int p, int k) __attribute__((always_inline)) {
    if (k < r1) {
      nq[p] = *reinterpret_cast<const vt*>(view_row<T>(a.qu_cache, b, h, k) + sub * V);
      nu[p] = *reinterpret_cast<const vt*>(view_row<T>(a.U, b, h, k) + sub * V);
      nk[p] = *reinterpret_cast<const vt*>(view_row<T>(a.kc_cache, b, h, k) + sub * V);
      nv[p] = *reinterpret_cast<const vt*>(view_row<T>(a.vc_cache, b, h, k) + sub * V);
      if (np > 0) ng[p] = *reinterpret_cast<const vec<float, 4>*>(gbase + (int64_t)k * kDecodeDefer);
    }
  };
#pragma unroll
  for (int p = 0; p < PF; ++p) request(p, r0 + grp + p * RPI);
  for (int base = r0; base < r1; base += PF * RPI) {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
    const int k = base + p * RPI + grp;
    const vt cq = nq[p], cu = nu[p], ck = nk[p], cv = nv[p];
    const vec<float, 4> g4 = ng[p];
    request(p, k + PF * RPI);
    if (k < r1) {
      float quk[V], uk[V], kck[V], vck[V];
      T* urow = view_row<T>(a.U, b, h, k) + sub * V;
#pragma unroll
      for (int e = 0; e < V; ++e) { quk[e] = (float)cq[e]; kck[e] = (float)ck[e]; vck[e] = (float)cv[e]; }
      u_unpack<T, V, UH>(cu, uk);
      // pending sources j > k first (none unless the write-back is deferred): their gates were
      // formed by the steps that appended them and wait in the row's side array
      float* grow = deferred ? gbase + (int64_t)k * kDecodeDefer : nullptr;
      if (np > 0) {
#pragma unroll
        for (int sl = 0; sl < kDecodeDefer; ++sl) {
          const int j = pbase + ((sl - pbase % kDecodeDefer + kDecodeDefer) % kDecodeDefer);
          const float gj = (j < t && j > k) ? g4[sl] : 0.f;   // rows appended inside the window have no gate for earlier tokens
#pragma unroll
          for (int e = 0; e < V; ++e) uk[e] = __builtin_fmaf(gj, pv[sl][e], uk[e]);
        }
      }
      float dg = 0.f;
#pragma unroll
      for (int e = 0; e < V; ++e) dg = __builtin_fmaf(quk[e], ku[e], dg);
      dg = group_sum<LPR>(dg);
      const float gate = sigmoid_l2(dg * c1);
#pragma unroll
      for (int e = 0; e < V; ++e) uk[e] = __builtin_fmaf(gate, vu[e], uk[e]);
      if (write_u) {
        // the lookahead key as later steps will see it: the stored (rounded) one when it is written now
        const vt unew = u_pack<T, V, UH>(uk);
        *reinterpret_cast<vt*>(urow) = unew;
        u_unpack<T, V, UH>(unew, uk);
      } else if (sub == 0) {
        grow[slot_t] = gate;   // the new token stays pending: its gate for this row
      }
      float dsu = 0.f, dsc = 0.f;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        dsu = __builtin_fmaf(qc[e], uk[e], dsu);
        dsc = __builtin_fmaf(qc[e], kck[e], dsc);
      }
      dsu = group_sum<LPR>(dsu);
      dsc = group_sum<LPR>(dsc);
      const float x = (dsc - dsu * sigmoid_l2(dsu * c1)) * c1;   // score in log2 units
      const float mn = fmaxf(m, x);
      const float al = fast_exp2(m - mn), p_ = fast_exp2(x - mn);
      l = l * al + p_;
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = __builtin_fmaf(p_, vck[e], acc[e] * al);
      m = mn;
    }
    }
  }
  (void)c0;
  // merge the row groups of the workgroup
#pragma unroll
  for (int e = 0; e < V; ++e) s_acc[grp][sub * V + e] = acc[e];
  if (sub == 0) { s_acc[grp][HD] = m; s_acc[grp][HD + 1] = l; }
  __syncthreads();
  float* part = a.part + ((int64_t)bh * a.splits + split) * (HD + 2);
  if (tid < HD) {
    float M = -INFINITY;
    for (int r = 0; r < RPI; ++r) M = fmaxf(M, s_acc[r][HD]);
    float out = 0.f, lsum = 0.f;
    for (int r = 0; r < RPI; ++r) {
      const float w = (s_acc[r][HD] == -INFINITY) ? 0.f : fast_exp2(s_acc[r][HD] - M);
      out = __builtin_fmaf(w, s_acc[r][tid], out);
      lsum = __builtin_fmaf(w, s_acc[r][HD + 1], lsum);
    }
    part[tid] = out;
    if (tid == 0) { part[HD] = M; part[HD + 1] = lsum; }
  }
}

// One wave per (b, h): merge the split partials, add row t, normalise, append the new rows.
template <typename T, int HD>
__global__ __launch_bounds__(64) void decode_finish_kernel(DecodeArgs a) {
  constexpr int EPL = (HD + 63) / 64;   // elements per lane
  const int bh = blockIdx.x, b = bh / a.H, h = bh % a.H;
  const int lane = threadIdx.x;
  const int t = a.t_dev != nullptr ? *a.t_dev : a.t;
  if (t < 0 || t >= a.capacity) return;   // only reachable with a device-side count: the cache is full
  const float c1 = a.scale * kLog2e;
  const float* part = a.part + (int64_t)bh * a.splits * (HD + 2);
  const T* qc = view_row<T>(a.qc, b, h, 0);
  const T* kc = view_row<T>(a.kc, b, h, 0);
  const T* vc = view_row<T>(a.vc, b, h, 0);
  const T* qu = view_row<T>(a.qu, b, h, 0);

  float dot = 0.f;
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    const int n = lane + 64 * e;
    if (n < HD) dot = __builtin_fmaf((float)qc[n], (float)kc[n], dot);
  }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) dot += __shfl_xor(dot, o);
  const float xt = dot * c1;            // row t: U_t = 0, so the lookahead term is silu(0) = 0

  // statistics of the partials: lane s holds split s (at most 64 splits), so the loads of all
  // splits are in flight together instead of one dependent load per loop iteration
  const int nsplit = t > 0 ? a.splits : 0;
  float ms_l = -INFINITY, ls_l = 0.f;
  if (lane < nsplit) {
    ms_l = part[lane * (HD + 2) + HD];
    ls_l = part[lane * (HD + 2) + HD + 1];
  }
  float M = ms_l;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) M = fmaxf(M, __shfl_xor(M, o));
  M = fmaxf(M, xt);
  const float w_l = (ms_l == -INFINITY) ? 0.f : fast_exp2(ms_l - M);
  float lsum = w_l * ls_l;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) lsum += __shfl_xor(lsum, o);
  const float pt = fast_exp2(xt - M);
  lsum += pt;
  float o[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    const int n = lane + 64 * e;
    o[e] = n < HD ? pt * (float)vc[n] : 0.f;
  }
  constexpr int SU = 8;   // partial rows loaded per batch
  for (int s0 = 0; s0 < nsplit; s0 += SU) {
    float v[SU][EPL];
#pragma unroll
    for (int u = 0; u < SU; ++u)
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const int n = lane + 64 * e;
        v[u][e] = (s0 + u < nsplit && n < HD) ? part[(s0 + u) * (HD + 2) + n] : 0.f;
      }
#pragma unroll
    for (int u = 0; u < SU; ++u) {
      const float w = __shfl(w_l, (s0 + u) & 63);   // 0 for lanes beyond nsplit
#pragma unroll
      for (int e = 0; e < EPL; ++e) o[e] = __builtin_fmaf(w, v[u][e], o[e]);
    }
  }
  const float inv = 1.f / lsum;
  const bool deferred = a.pend_vu.ptr != nullptr;
  const T* vu = view_row<T>(a.vu, b, h, 0);
  T* pvt = deferred ? view_row<T>(a.pend_vu, b, h, t % kDecodeDefer) : nullptr;
  T* out = view_row<T>(a.out, b, h, 0);
  T* Ut = view_row<T>(a.U, b, h, t);
  T* qut = view_row<T>(a.qu_cache, b, h, t);
  T* kct = view_row<T>(a.kc_cache, b, h, t);
  T* vct = view_row<T>(a.vc_cache, b, h, t);
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    const int n = lane + 64 * e;
    float quv = n < HD ? (float)qu[n] : 0.f, kcv = n < HD ? (float)kc[n] : 0.f;
    if (a.rotary) {   // element n and its pair partner n ^ 1 sit on neighbouring lanes
      const float qup = __shfl_xor(quv, 1), kcp = __shfl_xor(kcv, 1);
      const bool even = (n & 1) == 0;
      float q0 = even ? quv : qup, q1 = even ? qup : quv, k0 = even ? kcv : kcp, k1 = even ? kcp : kcv;
      CASTLE_ROPE_PAIR(q0, q1, (float)t, n / 2, HD, false);
      CASTLE_ROPE_PAIR(k0, k1, (float)t, n / 2, HD, false);
      quv = even ? q0 : q1;
      kcv = even ? k0 : k1;
    }
    if (n < HD) {
      out[n] = (T)(o[e] * inv);
      Ut[n] = (T)0.f;
      qut[n] = (T)quv;
      kct[n] = (T)kcv;
      vct[n] = vc[n];
    }
    if (deferred) {   // the new token joins the pending sources (rotated like the stream kernel uses it)
      float vuv = n < HD ? (float)vu[n] : 0.f;
      if (a.rotary) {
        const float vup = __shfl_xor(vuv, 1);
        const bool even = (n & 1) == 0;
        float v0 = even ? vuv : vup, v1 = even ? vup : vuv;
        CASTLE_ROPE_PAIR(v0, v1, (float)t, n / 2, HD, false);
        vuv = even ? v0 : v1;
      }
      if (n < HD) pvt[n] = (T)vuv;
    }
  }
}

// Folds the pending sources into the stored lookahead keys (rows 0 .. t-1), for a reader that wants
// the cache tensor U itself: U_k += sum over pending j > k of sigmoid(s qu_k . ku_j) vu_j.
template <typename T, int HD, bool UH>
__global__ __launch_bounds__(kThreads) void decode_flush_kernel(DecodeArgs a) {
  constexpr int V = elem_traits<T>::vec16;
  constexpr int LPR = HD / V;
  constexpr int RPI = kThreads / LPR;
  typedef vec<T, V> vt;
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const int t = a.t;
  const int grp = threadIdx.x / LPR, sub = threadIdx.x % LPR;
  const float c1 = a.scale * kLog2e;
  const int pbase = decode_base(a.base0, t);
  float pv[kDecodeDefer][V];
#pragma unroll
  for (int sl = 0; sl < kDecodeDefer; ++sl) {
#pragma unroll
    for (int e = 0; e < V; ++e) pv[sl][e] = 0.f;
    const int j = pbase + ((sl - pbase % kDecodeDefer + kDecodeDefer) % kDecodeDefer);
    if (j < t) load_f32<T, V>(view_row<T>(a.pend_vu, b, h, sl) + sub * V, pv[sl]);
  }
  (void)c1;
  for (int k = blockIdx.x * RPI + grp; k < t; k += gridDim.x * RPI) {
    float uk[V];
    T* urow = view_row<T>(a.U, b, h, k) + sub * V;
    u_unpack<T, V, UH>(*reinterpret_cast<const vt*>(urow), uk);
    const vec<float, 4> g4 = *reinterpret_cast<const vec<float, 4>*>(
        reinterpret_cast<const float*>(a.pend_gate.ptr) + (int64_t)b * a.pend_gate.sb + (int64_t)h * a.pend_gate.sh + (int64_t)k * kDecodeDefer);
#pragma unroll
    for (int sl = 0; sl < kDecodeDefer; ++sl) {
      const int j = pbase + ((sl - pbase % kDecodeDefer + kDecodeDefer) % kDecodeDefer);
      const float gj = (j < t && j > k) ? g4[sl] : 0.f;
#pragma unroll
      for (int e = 0; e < V; ++e) uk[e] = __builtin_fmaf(gj, pv[sl][e], uk[e]);
    }
    *reinterpret_cast<vt*>(urow) = u_pack<T, V, UH>(uk);
  }
}

template <typename T, int HD> static int launch_decode_t(const DecodeArgs& a, hipStream_t stream) {
  const int BH = a.B * a.H;
  if (a.t_dev != nullptr || a.t > 0) {
    ProfScope ps(kSlotDecodeStream, stream);
    if constexpr (__is_same(T, bf16_t)) {
      if (a.u_half) hipLaunchKernelGGL((decode_stream_kernel<T, HD, true>), dim3(a.splits, BH), dim3(kThreads), 0, stream, a);
      else hipLaunchKernelGGL((decode_stream_kernel<T, HD, false>), dim3(a.splits, BH), dim3(kThreads), 0, stream, a);
    } else {
      hipLaunchKernelGGL((decode_stream_kernel<T, HD, false>), dim3(a.splits, BH), dim3(kThreads), 0, stream, a);
    }
  }
  {
    ProfScope ps(kSlotDecodeFinish, stream);
    hipLaunchKernelGGL((decode_finish_kernel<T, HD>), dim3(BH), dim3(64), 0, stream, a);
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <typename T, int HD> static void launch_flush_t(const DecodeArgs& a, dim3 grid, hipStream_t stream) {
  if constexpr (__is_same(T, bf16_t)) {
    if (a.u_half) { hipLaunchKernelGGL((decode_flush_kernel<T, HD, true>), grid, dim3(kThreads), 0, stream, a); return; }
  }
  hipLaunchKernelGGL((decode_flush_kernel<T, HD, false>), grid, dim3(kThreads), 0, stream, a);
}
template <typename T> static int launch_flush_d(const DecodeArgs& a, hipStream_t stream) {
  const int BH = a.B * a.H;
  int gx = (640 + BH - 1) / BH;
  if (gx > 64) gx = 64;
  const dim3 grid(gx, BH);
  switch (a.d) {
    case 16: launch_flush_t<T, 16>(a, grid, stream); break;
    case 32: launch_flush_t<T, 32>(a, grid, stream); break;
    case 64: launch_flush_t<T, 64>(a, grid, stream); break;
    case 128: launch_flush_t<T, 128>(a, grid, stream); break;
    default: return -2;
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

int launch_decode_flush(const DecodeArgs& a, int dtype, hipStream_t stream) {
  switch (dtype) {
    case 0: return launch_flush_d<float>(a, stream);
    case 1: return launch_flush_d<bf16_t>(a, stream);
    case 2: return launch_flush_d<fp16_t>(a, stream);
    default: return -1;
  }
}

template <typename T> static int launch_decode_d(const DecodeArgs& a, hipStream_t stream) {
  switch (a.d) {
    case 16: return launch_decode_t<T, 16>(a, stream);
    case 32: return launch_decode_t<T, 32>(a, stream);
    case 64: return launch_decode_t<T, 64>(a, stream);
    case 128: return launch_decode_t<T, 128>(a, stream);
    default: return -2;
  }
}

int launch_decode(const DecodeArgs& a, int dtype, hipStream_t stream) {
  switch (dtype) {
    case 0: return launch_decode_d<float>(a, stream);
    case 1: return launch_decode_d<bf16_t>(a, stream);
    case 2: return launch_decode_d<fp16_t>(a, stream);
    default: return -1;
  }
}

// ---------------------------------------------------------------------------
// Out-of-place rotary embedding of one (B, H, L, d) view: dst = R(pos0 + row) src.
template <typename T, int HD>
__global__ __launch_bounds__(kThreads) void rope_kernel(View4 src, View4 dst, int H, int L, int pos0) {
  constexpr int V = elem_traits<T>::vec16;
  constexpr int VPR = HD / V;
  const int bh = blockIdx.y, b = bh / H, h = bh % H;
  const int64_t piece = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int64_t row = piece / VPR;
  const int cv = (int)(piece % VPR);
  if (row >= L) return;
  vec<float, V> f = __builtin_convertvector(*reinterpret_cast<const vec<T, V>*>(view_row<T>(src, b, h, row) + cv * V), vec<float, V>);
#pragma unroll
  for (int e = 0; e < V / 2; ++e) CASTLE_ROPE_PAIR(f[2 * e], f[2 * e + 1], (float)(pos0 + row), cv * (V / 2) + e, HD, false);
  *reinterpret_cast<vec<T, V>*>(view_row<T>(dst, b, h, row) + cv * V) = __builtin_convertvector(f, vec<T, V>);
}

template <typename T> static int launch_rope_d(const View4& src, const View4& dst, int B, int H, int L, int d, int pos0, hipStream_t stream) {
  const int pieces_per_row = d / elem_traits<T>::vec16;
  const dim3 grid((unsigned)(((int64_t)L * pieces_per_row + kThreads - 1) / kThreads), B * H);
  switch (d) {
    case 16: hipLaunchKernelGGL((rope_kernel<T, 16>), grid, dim3(kThreads), 0, stream, src, dst, H, L, pos0); break;
    case 32: hipLaunchKernelGGL((rope_kernel<T, 32>), grid, dim3(kThreads), 0, stream, src, dst, H, L, pos0); break;
    case 64: hipLaunchKernelGGL((rope_kernel<T, 64>), grid, dim3(kThreads), 0, stream, src, dst, H, L, pos0); break;
    case 128: hipLaunchKernelGGL((rope_kernel<T, 128>), grid, dim3(kThreads), 0, stream, src, dst, H, L, pos0); break;
    default: return -2;
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

int launch_rope(const View4& src, const View4& dst, int B, int H, int L, int d, int dtype, int pos0, hipStream_t stream) {
  switch (dtype) {
    case 0: return launch_rope_d<float>(src, dst, B, H, L, d, pos0, stream);
    case 1: return launch_rope_d<bf16_t>(src, dst, B, H, L, d, pos0, stream);
    case 2: return launch_rope_d<fp16_t>(src, dst, B, H, L, d, pos0, stream);
    default: return -1;
  }
}

// ---------------------------------------------------------------------------
// y[M, N] = x[M, K] w[N, K]^T for the few rows of a decode step (M = batch): the two projections
// around the cached step (lookahead_keys_attention.py:99, 209 with seq_len == 1).  A library GEMM
// spends most of its ~8 us here on one 32-row tile per workgroup walking K serially; this kernel
// gives every 32 x 32 output tile to one workgroup of 8 waves that split K, so each wave issues all
// its operand loads at once (straight from global memory, rows of x and w are K-contiguous, which is
// the MFMA operand layout), runs a handful of MFMAs and the partial tiles are summed through LDS.
constexpr int kLinWaves = 8;
// Optional work around the product (all of it per output row, so it costs one pass less each):
//   norm_w   RMS normalisation of the x rows in front: y = ((x / rms(x)) * norm_w) w^T.  The weight
//            goes into the operand, the 1 / rms factor (a per-row scalar) onto the accumulated sum;
//            the sums of squares are collected from the fragments the product loads anyway.
//   act      1: GELU (erf form) of the sum
//   res      a tensor of the output's shape added at the end
template <typename T>
__global__ __launch_bounds__(64 * kLinWaves) void small_linear_kernel(const T* x, const T* w, T* y, int M, int N, int K,
                                                                       int64_t ldx, int64_t ldw, int64_t ldy,
                                                                       const T* norm_w, float eps, int act,
                                                                       const T* res, int64_t ldr) {
  static_assert(sizeof(T) == 2, "16-bit operands");
  constexpr int MAXS = 8;   // 16-deep steps a wave handles per pass
  __shared__ float red[kLinWaves][32][33];
  __shared__ float ssq[kLinWaves][32];
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const int n0 = blockIdx.x * 32, m0 = blockIdx.y * 32;
  const int steps = (K + 15) / 16;
  const int per = (steps + kLinWaves - 1) / kLinWaves;
  const bool row_ok = m0 + c < M, col_ok = n0 + c < N;
  const T* xr = x + (int64_t)(m0 + c) * ldx;
  const T* wr = w + (int64_t)(n0 + c) * ldw;
  acc_t acc;
  zero(acc);
  float sq = 0.f;
  for (int s0 = wave * per; s0 < min(steps, (wave + 1) * per); s0 += MAXS) {
    frag<T> fa[MAXS], fb[MAXS];
#pragma unroll
    for (int u = 0; u < MAXS; ++u) {
      const int kk = 16 * (s0 + u) + 8 * g;
      const bool in = s0 + u < min(steps, (wave + 1) * per) && kk < K;   // K is a multiple of 8
      fa[u] = (in && row_ok) ? *reinterpret_cast<const frag_mem<T>*>(xr + kk) : zero_frag<T>();
      fb[u] = (in && col_ok) ? *reinterpret_cast<const frag_mem<T>*>(wr + kk) : zero_frag<T>();
      if (norm_w != nullptr) {
        const frag<T> fg = in ? *reinterpret_cast<const frag_mem<T>*>(norm_w + kk) : zero_frag<T>();
        const vec<float, 8> xv = __builtin_convertvector(fa[u], vec<float, 8>);
        const vec<float, 8> gv = __builtin_convertvector(fg, vec<float, 8>);
#pragma unroll
        for (int e = 0; e < 8; ++e) sq = __builtin_fmaf(xv[e], xv[e], sq);
        fa[u] = __builtin_convertvector(xv * gv, frag<T>);
      }
    }
#pragma unroll
    for (int u = 0; u < MAXS; ++u) mma(acc, fa[u], fb[u]);
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) red[wave][acc_row(r, g)][c] = acc[r];
  if (norm_w != nullptr) {
    sq += __shfl_xor(sq, 32);   // the two halves of a row's 16-deep steps
    if (g == 0) ssq[wave][c] = sq;
  }
  __syncthreads();
  // 1024 outputs, 512 threads: two neighbouring columns each
  const int e = 2 * threadIdx.x, row = e / 32, col = e % 32;
  float s0 = 0.f, s1 = 0.f;
#pragma unroll
  for (int v = 0; v < kLinWaves; ++v) { s0 += red[v][row][col]; s1 += red[v][row][col + 1]; }
  if (norm_w != nullptr) {
    float t = 0.f;
#pragma unroll
    for (int v = 0; v < kLinWaves; ++v) t += ssq[v][row];
    const float rstd = __builtin_amdgcn_rsqf(t / (float)K + eps);
    s0 *= rstd;
    s1 *= rstd;
  }
  if (act == 1) {
    s0 = 0.5f * s0 * (1.f + erff(s0 * 0.70710678f));
    s1 = 0.5f * s1 * (1.f + erff(s1 * 0.70710678f));
  }
  if (m0 + row < M) {
    T* dst = y + (int64_t)(m0 + row) * ldy + n0 + col;
    const T* rsrc = res != nullptr ? res + (int64_t)(m0 + row) * ldr + n0 + col : nullptr;
    if (n0 + col + 1 < N) {
      if (rsrc != nullptr) {
        const vec<T, 2> rv = *reinterpret_cast<const vec<T, 2>*>(rsrc);
        s0 += (float)rv[0];
        s1 += (float)rv[1];
      }
      vec<T, 2> o = {(T)s0, (T)s1};
      *reinterpret_cast<vec<T, 2>*>(dst) = o;
    } else if (n0 + col < N) {
      if (rsrc != nullptr) s0 += (float)rsrc[0];
      dst[0] = (T)s0;
    }
  }
}
int launch_small_linear(const void* x, const void* w, void* y, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldy,
                        int dtype, const void* norm_w, float eps, int act, const void* res, int64_t ldr, hipStream_t stream) {
  const dim3 grid((N + 31) / 32, (M + 31) / 32), block(64 * kLinWaves);
  if (dtype == 1)
    hipLaunchKernelGGL((small_linear_kernel<bf16_t>), grid, block, 0, stream, static_cast<const bf16_t*>(x),
                       static_cast<const bf16_t*>(w), static_cast<bf16_t*>(y), M, N, K, ldx, ldw, ldy,
                       static_cast<const bf16_t*>(norm_w), eps, act, static_cast<const bf16_t*>(res), ldr);
  else if (dtype == 2)
    hipLaunchKernelGGL((small_linear_kernel<fp16_t>), grid, block, 0, stream, static_cast<const fp16_t*>(x),
                       static_cast<const fp16_t*>(w), static_cast<fp16_t*>(y), M, N, K, ldx, ldw, ldy,
                       static_cast<const fp16_t*>(norm_w), eps, act, static_cast<const fp16_t*>(res), ldr);
  else
    return -1;
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

// ---------------------------------------------------------------------------
// Partial-result buffer of the entry point that allocates nothing: one array per GPU, part of the
// loaded code object, alive until the process ends.  Host code never uses the array's name as an
// address (on the host it is only a stand-in for the symbol): the device address is looked up
// once per device and handed to the kernels like any other workspace pointer.
static __device__ __align__(256) unsigned char scratch[kDecodeStaticScratchBytes];

int decode_static_scratch(float** ptr) {
  static std::mutex mu;
  static void* per_device[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -3;
  std::lock_guard<std::mutex> lock(mu);
  if (per_device[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return -3;
    per_device[dev] = p;
  }
  *ptr = static_cast<float*>(per_device[dev]);
  return 0;
}

// rows of one (b, h) handled per workgroup iteration, needed by the host to size `splits`
int decode_pick_splits(int BH, int t) {
  if (t <= 0) return 1;
  int want = (CASTLE_DEC_WGS + BH - 1) / BH;           // 2-3 workgroups per CU: measured 6.3 TB/s at 512-768 workgroups, 6.0 at 2048, 4.5 at 256
  int max_by_rows = (t + 63) / 64;          // at least 64 rows per workgroup
  int s = want < max_by_rows ? want : max_by_rows;
  if (s < 1) s = 1;
  if (s > 64) s = 64;
  return s;
}

}  // namespace castle
