// CASTLE parallel backward for gfx950: reverse-state form, score tiles recomputed.
//
// Gradients follow the closed forms the reference's backward kernel evaluates
// (lookahead_keys_attention_triton.py:333-401) with the O(L^3) loops replaced by a
// reverse state per key:  G_k(I) = sum_{i >= (I+1)*64} dSu[i,k] qc_i.
//
//   delta_kernel      delta_i = rowsum(dO_i * O_i)
//   bwd_key_kernel    key-stationary, 128 keys per workgroup (32 per wave, keys on lanes),
//                     query blocks swept from the last one down:
//                     dVc, dKc, dQu accumulate in registers, G is carried in registers and
//                     stored as snapshot gsnap[I][k] before block I is folded in.
//   bwd_query_kernel  query-stationary, 128 rows per workgroup (32 per wave, rows on lanes),
//                     keys streamed in chunks of 32: dQc (rows as queries) and dKu, dVu
//                     (rows as lookahead sources), using the forward snapshots usnap and gsnap.
//
// Units (s = softmax scale, c1 = s log2 e).  As in the forward pass the resident query operand is
// Qc' = c1 Qc, the stored T blocks are T' = c1 tril(Qc Vu^T) and the resident gate operand is
// multiplied by -c1, so scores come out of the MFMA in log2 units.  dS and dSu are the gradients
// with respect to the TRUE scores.  Everything that is built from Qc' or T' carries a factor c1:
//   G' = sum dSu^T Qc' = c1 G,   dA' = dSu^T T' + G' Vu^T = c1 dA,   dZ' = dA' A (1 - A)
// and the outputs are rescaled once at the end:
//   dKc = ln2 (dS^T Qc')      dVc = P^T dO              dQu = s ln2 (dZ' Ku)
//   dQc = s (dS Kc + dSu U + dT Vu)   dKu = s ln2 (dZ'^T Qu)   dVu = ln2 (A^T G' + dT^T Qc')
#include "castle_tiles.h"
#include "castle_params.h"
#include "castle_profile.h"

namespace castle {

extern __shared__ __attribute__((aligned(16))) unsigned char castle_smem[];

template <typename T> __device__ __forceinline__ const T* head_ptr(const View4& v, int b, int h) {
  return reinterpret_cast<const T*>(v.ptr) + (int64_t)b * v.sb + (int64_t)h * v.sh;
}
template <typename T> __device__ __forceinline__ T* head_ptr_mut(const View4& v, int b, int h) {
  return reinterpret_cast<T*>(v.ptr) + (int64_t)b * v.sb + (int64_t)h * v.sh;
}

// Operand whose FREE index sits on lanes, read from data stored [contraction][free].
// 16-bit types read a transposed LDS copy tc[free][contraction]; fp32 gathers from the
// row-major tile rm[contraction][free] (free >= free_limit reads as zero).
template <typename T>
__device__ __forceinline__ frag<T> ld_tr_chain(const T* tc, int ldt, const T* rm, int ldr, int free_idx, int free_limit, int contr0, int g) {
  if constexpr (sizeof(T) == 2) {
    return ld_chain<T>(tc, ldt, free_idx, contr0, g);
  } else {
    frag<T> f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = contr0 + 8 * (e >> 2) + 4 * g + (e & 3);
      f[e] = free_idx < free_limit ? rm[j * ldr + free_idx] : (T)0.f;
    }
    return f;
  }
}
template <typename T>
__device__ __forceinline__ frag<T> ld_tr_nat(const T* tc, int ldt, const T* rm, int ldr, int free_idx, int free_limit, int contr0, int g) {
  if constexpr (sizeof(T) == 2) {
    return ld_nat<T>(tc, ldt, free_idx, contr0 + 8 * g);
  } else {
    frag<T> f;
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = free_idx < free_limit ? rm[(contr0 + 8 * g + e) * ldr + free_idx] : (T)0.f;
    return f;
  }
}

struct Carver {
  unsigned char* p;
  template <typename U> __device__ __forceinline__ U* take(int count) {
    U* r = reinterpret_cast<U*>(p);
    p += (count * (int)sizeof(U) + 15) / 16 * 16;
    return r;
  }
};
constexpr int a16(int bytes) { return (bytes + 15) / 16 * 16; }

// [n rows, lanes] accumulator tiles -> (row = lane index, 4 consecutive n) stores, scaled
template <typename T, int HD, int NT>   // T: element type of the destination tensor
__device__ __forceinline__ void store_rows(T* dst_row, acc_t (&acc)[NT], float mul, int g) {
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nt][r] *= mul;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = 32 * nt + 8 * q + 4 * g;
      if (n < HD) st4<T>(dst_row + n, pack4<T>(acc[nt], q));
    }
  }
}

// ---------------------------------------------------------------------------
template <typename T, int HD>
__global__ __launch_bounds__(kThreads) void delta_kernel(BwdArgs a) {
  constexpr int V = elem_traits<T>::vec16;
  constexpr int LPR = HD / V;
  constexpr int RPB = kThreads / LPR;
  typedef vec<T, V> vt;
  const int bh = blockIdx.y, b = bh / a.s.H, h = bh % a.s.H;
  const int grp = threadIdx.x / LPR, sub = threadIdx.x % LPR;
  const int64_t i = (int64_t)blockIdx.x * RPB + grp;
  if (i >= a.s.Lp) return;
  float acc = 0.f;
  if (i < a.s.L) {
    vt o = *reinterpret_cast<const vt*>(head_ptr<T>(a.out, b, h) + i * a.out.sl + sub * V);
    vt d = *reinterpret_cast<const vt*>(head_ptr<T>(a.dout, b, h) + i * a.dout.sl + sub * V);
#pragma unroll
    for (int e = 0; e < V; ++e) acc = __builtin_fmaf((float)o[e], (float)d[e], acc);
  }
#pragma unroll
  for (int o = 1; o < LPR; o <<= 1) acc += __shfl_xor(acc, o);
  if (sub == 0) a.delta[(int64_t)bh * a.s.Lp + i] = acc;
}

// ---------------------------------------------------------------------------
template <typename T, int HD> constexpr int bwd_key_lds_bytes() {
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr bool TC = sizeof(T) == 2;
  int b = 0;
  b += 3 * a16((int)sizeof(T) * kNB * lds_ld<T>(HD));           // qc, do, ku
  b += a16((int)sizeof(T) * kNB * lds_ld_chain<T>(HD));         // vu
  b += a16((int)sizeof(T) * kNB * lds_ld_chain<T>(kNB));        // T
  if (TC) {
    b += 3 * a16((int)sizeof(T) * HDP * lds_ld_chain<T>(kNB));  // qc^T, do^T, ku^T
    b += a16((int)sizeof(T) * kNB * lds_ld_chain<T>(kNB));      // T^T
  }
  b += 2 * a16(4 * kNB);                                  // lse, delta
  return b;
}

template <typename T, typename TI, int HD>
__global__ __launch_bounds__(kThreads, 1) void bwd_key_kernel(BwdArgs a) {
  constexpr int KS = HD / 16;
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr int NT = HDP / 32;
  constexpr int BT = kNB / 32;   // 32-row sub-tiles per block
  constexpr bool TC = sizeof(T) == 2;
  constexpr int LDK = lds_ld<T>(HD), LDU = lds_ld_chain<T>(HD), LDV = lds_ld_chain<T>(kNB), LDT = lds_ld_chain<T>(kNB);

  Carver cv{castle_smem};
  T* s_qc = cv.take<T>(kNB * LDK);
  T* s_do = cv.take<T>(kNB * LDK);
  T* s_ku = cv.take<T>(kNB * LDK);
  T* s_vu = cv.take<T>(kNB * LDU);
  T* s_t = cv.take<T>(kNB * LDT);
  T* s_qct = s_qc; T* s_dot = s_do; T* s_kut = s_ku; T* s_tt = s_t;
  if constexpr (TC) {
    s_qct = cv.take<T>(HDP * LDV);
    s_dot = cv.take<T>(HDP * LDV);
    s_kut = cv.take<T>(HDP * LDV);
    s_tt = cv.take<T>(kNB * LDT);
  }
  float* s_lse = cv.take<float>(kNB);
  float* s_delta = cv.take<float>(kNB);

  int kb, bh;   // key group 0 meets every query block: rank order = kb
  work_item(a.s.B * a.s.H, kb, bh);
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const int L = a.s.L;
  const float c0 = a.s.scale, c1 = a.s.scale * kLog2e;
  const int kw0 = kb * 128 + 32 * wave;
  const int k = kw0 + c;
  const int Iw = kw0 / kNB;
  const int sgroup = wave >> 1, slt = threadIdx.x & 127;   // staging group and index inside it
  const TI* qc = head_ptr<TI>(a.qc, b, h);
  const TI* kc = head_ptr<TI>(a.kc, b, h);
  const TI* vc = head_ptr<TI>(a.vc, b, h);
  const TI* qu = head_ptr<TI>(a.qu, b, h);
  const TI* ku = head_ptr<TI>(a.ku, b, h);
  const TI* vu = head_ptr<TI>(a.vu, b, h);
  const TI* dout = head_ptr<TI>(a.dout, b, h);
  const T* tb = reinterpret_cast<const T*>(a.ws.t_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* ttb = reinterpret_cast<const T*>(a.ws.tt_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* usnap = reinterpret_cast<const T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  T* gsnap = reinterpret_cast<T*>(a.gsnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  const float* lse = a.ws.lse + (int64_t)bh * a.s.Lp;
  const float* delta = a.delta + (int64_t)bh * a.s.Lp;

  frag<T> fkc[KS], fvc[KS], fqu[KS], fub[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    fkc[s] = ldg_nat<T, TI>(kc, a.kc.sl, k, 16 * s + 8 * g, k < L);
    fvc[s] = ldg_nat<T, TI>(vc, a.vc.sl, k, 16 * s + 8 * g, k < L);
    fqu[s] = ldg_nat_scaled<T, TI>(qu, a.qu.sl, k, 16 * s + 8 * g, k < L, -c1);
    fub[s] = zero_frag<T>();
  }
  acc_t dvc[NT], dkc[NT], dqu[NT], G[NT];   // [n rows, k lanes]
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) { zero(dvc[nt]); zero(dkc[nt]); zero(dqu[nt]); zero(G[nt]); }
  if (TC && HDP > HD) {
    lds_zero(s_qct + HD * LDV, (HDP - HD) * LDV);
    lds_zero(s_dot + HD * LDV, (HDP - HD) * LDV);
    lds_zero(s_kut + HD * LDV, (HDP - HD) * LDV);
  }

  PatchStage<T, TI, kNB, HD, 128> pa, pb;
  PatchStage<T, T, kNB, kNB, 128> pt;
  auto stage_load = [&](int I) __attribute__((always_inline)) {
    const int64_t r0 = (int64_t)I * kNB;
    if (sgroup == 0) {
      pa.load(slt, qc, a.qc.sl, r0, L);
      pb.load(slt, ku, a.ku.sl, r0, L);
      pt.load(slt, tb, kNB, r0, (int64_t)1 << 40);
    } else {
      pa.load(slt, dout, a.dout.sl, r0, L);
      pb.load(slt, vu, a.vu.sl, r0, L);
      if constexpr (TC) pt.load(slt, ttb, kNB, r0, (int64_t)1 << 40);
    }
  };
  auto stage_store = [&]() __attribute__((always_inline)) {
    if (sgroup == 0) {
      pa.store_rows(slt, s_qc, LDK, c1);
      if constexpr (TC) pa.store_cols(slt, s_qct, LDV, c1);
      pb.store_rows(slt, s_ku, LDK);
      if constexpr (TC) pb.store_cols(slt, s_kut, LDV);
      pt.template store_rows<true>(slt, s_t, LDT);
    } else {
      pa.store_rows(slt, s_do, LDK);
      if constexpr (TC) pa.store_cols(slt, s_dot, LDV);
      pb.template store_rows<true>(slt, s_vu, LDU);
      if constexpr (TC) pt.template store_rows<true>(slt, s_tt, LDT);
    }
  };

  const int I0 = (kb * 128) / kNB;
  stage_load(a.s.nblk - 1);
  for (int I = a.s.nblk - 1; I >= I0; --I) {
    const bool active = I >= Iw;
    if (active && I <= a.s.nblk - 2) {   // reverse state as of block I
      T* dst = gsnap + (gsnap_off(I) + k) * HD;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = 32 * nt + 8 * q + 4 * g;
          if (n < HD) st4<T>(dst + n, pack4<T>(G[nt], q));
        }
    }
    if (I > Iw) {
#pragma unroll
      for (int s = 0; s < KS; ++s) fub[s] = ldg_nat<T>(usnap + usnap_off(I) * HD, HD, k, 16 * s + 8 * g, true);
    }
    __syncthreads();
    const int64_t r0 = (int64_t)I * kNB;
    // two thread groups (waves 0-1 / waves 2-3) stage three tiles each from the registers the
    // previous iteration filled, then issue the loads of the next block
    stage_store();
    if (I > I0) stage_load(I - 1);
    if (threadIdx.x < kNB) {
      const int64_t i = r0 + threadIdx.x;
      s_lse[threadIdx.x] = i < L ? lse[i] * kLog2e : INFINITY;
      s_delta[threadIdx.x] = i < L ? delta[i] : 0.f;
    }
    __syncthreads();
    if (!active) continue;

    // (a) gate tiles A^T[j rows, k lanes] for the whole source block
    acc_t aT[BT];
    frag<T> fa[BT][2];
#pragma unroll
    for (int jt = 0; jt < BT; ++jt) {
      zero(aT[jt]);
#pragma unroll
      for (int s = 0; s < KS; ++s) mma(aT[jt], ld_nat<T>(s_ku, LDK, 32 * jt + c, 16 * s + 8 * g), fqu[s]);
      const int j0 = I * kNB + 32 * jt;
#pragma unroll
      for (int r = 0; r < 16; ++r) aT[jt][r] = fast_rcp(1.f + fast_exp2(aT[jt][r]));
      if (j0 <= kw0 + 31) {   // tile touches the diagonal: keep j > k only
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (j0 + acc_row(r, g) <= k) aT[jt][r] = 0.f;
      }
      fa[jt][0] = chain<T>(aT[jt], 0);
      fa[jt][1] = chain<T>(aT[jt], 1);
    }
    // (b) dA^T[j rows, k lanes], second term first: G (before this block) times Vu^T
    acc_t dA[BT];
#pragma unroll
    for (int jt = 0; jt < BT; ++jt) {
      zero(dA[jt]);
#pragma unroll
      for (int s = 0; s < KS; ++s)
        mma(dA[jt], ld_chain<T>(s_vu, LDU, 32 * jt + c, 16 * s, g), chain<T>(G[s / 2], s % 2));
    }
    // (c) query sub-tiles of the block
#pragma unroll
    for (int it = 0; it < BT; ++it) {
      const int i0 = I * kNB + 32 * it;
      if (i0 + 31 < kw0) continue;   // every query precedes every key of this wave
      acc_t sc, su, dp;
      zero(sc); zero(su); zero(dp);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const frag<T> fq = ld_nat<T>(s_qc, LDK, 32 * it + c, 16 * s + 8 * g);
        mma(sc, fq, fkc[s]);
        if (I > Iw) mma(su, fq, fub[s]);
        mma(dp, ld_nat<T>(s_do, LDK, 32 * it + c, 16 * s + 8 * g), fvc[s]);
      }
#pragma unroll
      for (int jt = 0; jt < BT; ++jt) {
        if (jt > it) continue;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) mma(su, ld_chain<T>(s_t, LDT, 32 * it + c, 32 * jt + 16 * s2, g), fa[jt][s2]);
      }
      acc_t ds, dsu;
      const bool diag = i0 < kw0 + 31;   // tile touches the diagonal
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int il = 32 * it + acc_row(r, g);
        const float sg = fast_rcp(1.f + fast_exp2(-su[r]));
        const float x = __builtin_fmaf(-su[r], sg, sc[r]);
        float p = fast_exp2(x - s_lse[il]);
        if (diag && I * kNB + il < k) p = 0.f;
        const float dsv = p * (dp[r] - s_delta[il]);
        const float y = su[r] * kLn2;                     // true Su
        const float t = __builtin_fmaf(-y, sg, y);        // y (1 - sigmoid)
        const float sp = __builtin_fmaf(sg, t, sg);       // silu'(y)
        sc[r] = p;
        ds[r] = dsv;
        dsu[r] = -dsv * sp;
      }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const frag<T> fp = chain<T>(sc, s2), fds = chain<T>(ds, s2), fdsu = chain<T>(dsu, s2);
        const int ic = 32 * it + 16 * s2;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const frag<T> fdot = ld_tr_chain<T>(s_dot, LDV, s_do, LDK, 32 * nt + c, HD, ic, g);
          const frag<T> fqct = ld_tr_chain<T>(s_qct, LDV, s_qc, LDK, 32 * nt + c, HD, ic, g);
          mma(dvc[nt], fdot, fp);
          mma(dkc[nt], fqct, fds);
          mma(G[nt], fqct, fdsu);
        }
#pragma unroll
        for (int jt = 0; jt < BT; ++jt) {
          if (jt > it) continue;
          mma(dA[jt], ld_tr_chain<T>(s_tt, LDT, s_t, LDT, 32 * jt + c, kNB, ic, g), fdsu);
        }
      }
    }
    // (d) dZ^T = dA^T * A (1 - A)  ->  dQu
#pragma unroll
    for (int jt = 0; jt < BT; ++jt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) dA[jt][r] *= aT[jt][r] * (1.f - aT[jt][r]);
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const frag<T> fdz = chain<T>(dA[jt], s2);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          mma(dqu[nt], ld_tr_chain<T>(s_kut, LDV, s_ku, LDK, 32 * nt + c, HD, 32 * jt + 16 * s2, g), fdz);
      }
    }
  }
  if (k < L) {
    store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dkc, b, h) + (int64_t)k * a.dkc.sl, dkc, kLn2, g);
    store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dvc, b, h) + (int64_t)k * a.dvc.sl, dvc, 1.f, g);
    store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dqu, b, h) + (int64_t)k * a.dqu.sl, dqu, c0 * kLn2, g);
  }
}

// ---------------------------------------------------------------------------
constexpr int kCK = 32;   // keys per chunk in the query-stationary backward

template <typename T, int HD> constexpr int bwd_query_lds_bytes() {
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr bool TC = sizeof(T) == 2;
  int b = 0;
  b += 7 * a16((int)sizeof(T) * kCK * lds_ld<T>(HD));            // kc, vc, qu, ub[2], g[2]
  if (TC) b += 6 * a16((int)sizeof(T) * HDP * lds_ld_chain<T>(kCK));   // kc^T, qu^T, ub^T[2], g^T[2]
  b += 2 * a16((int)sizeof(T) * kCK * lds_ld<T>(128));                 // A, dSu
  if (TC) b += a16((int)sizeof(T) * 128 * lds_ld_chain<T>(kCK));       // A^T
  // epilogue (reuses the same memory): vu[2], qc[2], vu^T[2], qc^T[2], dT[2]
  int e = 0;
  e += 4 * a16((int)sizeof(T) * kNB * lds_ld<T>(HD));
  if (TC) e += 2 * a16((int)sizeof(T) * HDP * lds_ld_chain<T>(kNB)) + 2 * a16((int)sizeof(T) * HDP * lds_ld<T>(kNB));
  e += 2 * a16((int)sizeof(T) * kNB * lds_ld<T>(kNB));
  return b > e ? b : e;
}

template <typename T, typename TI, int HD>
__global__ __launch_bounds__(kThreads, 1) void bwd_query_kernel(BwdArgs a) {
  constexpr int KS = HD / 16;
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr int NT = HDP / 32;
  constexpr int BT = kNB / 32;
  constexpr int TS = kNB / 16;   // 16-deep steps across a block
  constexpr int QB = 128;
  constexpr int NQ = QB / kNB;
  constexpr bool TC = sizeof(T) == 2;
  constexpr int LDK = lds_ld<T>(HD), LDC = lds_ld_chain<T>(kCK), LDA = lds_ld<T>(QB);
  constexpr int LDV = lds_ld_chain<T>(kNB), LDQ = lds_ld<T>(kNB), LDT = lds_ld<T>(kNB);

  Carver cv{castle_smem};
  T* s_kc = cv.take<T>(kCK * LDK);
  T* s_vc = cv.take<T>(kCK * LDK);
  T* s_qu = cv.take<T>(kCK * LDK);
  T* s_ub[NQ]; T* s_g[NQ];
  for (int q = 0; q < NQ; ++q) s_ub[q] = cv.take<T>(kCK * LDK);
  for (int q = 0; q < NQ; ++q) s_g[q] = cv.take<T>(kCK * LDK);
  T* s_kct = s_kc; T* s_qut = s_qu; T* s_ubt[NQ]; T* s_gt[NQ];
  for (int q = 0; q < NQ; ++q) { s_ubt[q] = s_ub[q]; s_gt[q] = s_g[q]; }
  if constexpr (TC) {
    s_kct = cv.take<T>(HDP * LDC);
    s_qut = cv.take<T>(HDP * LDC);
    for (int q = 0; q < NQ; ++q) s_ubt[q] = cv.take<T>(HDP * LDC);
    for (int q = 0; q < NQ; ++q) s_gt[q] = cv.take<T>(HDP * LDC);
  }
  T* s_a = cv.take<T>(kCK * LDA);
  T* s_dsu = cv.take<T>(kCK * LDA);
  T* s_at = s_a;
  if constexpr (TC) s_at = cv.take<T>(QB * LDC);

  int rank, bh;
  work_item(a.s.B * a.s.H, rank, bh);
  const int qb = a.s.Lp / 128 - 1 - rank;   // the last row block meets the most keys
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const int L = a.s.L;
  const float c0 = a.s.scale, c1 = a.s.scale * kLog2e;
  const int i0w = qb * QB + 32 * wave;
  const int i = i0w + c;                      // this lane's row: a query in phase 1, a source in phase 2
  const int Ifirst = (qb * QB) / kNB;
  const int Iw = i0w / kNB;
  const int qw = Iw - Ifirst;                 // which of the workgroup's blocks
  const int jw = 32 * wave;                   // columns of this wave inside the 128-wide tiles
  const int cb = (jw / kNB) * kNB;            // first column of its block
  const int lw = jw % kNB;                    // offset of the wave inside its block
  const int nintra = (lw + 32) / 16;          // steps covering sources j <= i
  const int ifirst = lw / 16;                 // first step covering queries i >= j
  const bool has_g = Iw <= a.s.nblk - 2;

  const TI* qc = head_ptr<TI>(a.qc, b, h);
  const TI* kc = head_ptr<TI>(a.kc, b, h);
  const TI* vc = head_ptr<TI>(a.vc, b, h);
  const TI* qu = head_ptr<TI>(a.qu, b, h);
  const TI* ku = head_ptr<TI>(a.ku, b, h);
  const TI* vu = head_ptr<TI>(a.vu, b, h);
  const TI* dout = head_ptr<TI>(a.dout, b, h);
  const T* tb = reinterpret_cast<const T*>(a.ws.t_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* ttb = reinterpret_cast<const T*>(a.ws.tt_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* usnap = reinterpret_cast<const T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  const T* gsnap = reinterpret_cast<const T*>(a.gsnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;

  frag<T> fqc[KS], fdo[KS], fku[KS], fvu[KS], ft[TS], ftt[TS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    fqc[s] = ldg_nat_scaled<T, TI>(qc, a.qc.sl, i, 16 * s + 8 * g, i < L, c1);
    fdo[s] = ldg_nat<T, TI>(dout, a.dout.sl, i, 16 * s + 8 * g, i < L);
    fku[s] = ldg_nat_scaled<T, TI>(ku, a.ku.sl, i, 16 * s + 8 * g, i < L, -c1);
    fvu[s] = ldg_nat<T, TI>(vu, a.vu.sl, i, 16 * s + 8 * g, i < L);
  }
#pragma unroll
  for (int s = 0; s < TS; ++s) {
    ft[s] = ldg_nat<T>(tb, kNB, i, 16 * s + 8 * g, s < nintra);
    ftt[s] = ldg_nat<T>(ttb, kNB, i, 16 * s + 8 * g, s >= ifirst);
  }
  const float lse2 = i < L ? a.ws.lse[(int64_t)bh * a.s.Lp + i] * kLog2e : INFINITY;
  const float dlt = i < L ? a.delta[(int64_t)bh * a.s.Lp + i] : 0.f;

  acc_t dqc[NT], dku[NT], dvu[NT];   // [n rows, row-of-this-lane]
  acc_t dtacc[BT];                   // [j rows (block local), i lanes]
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) { zero(dqc[nt]); zero(dku[nt]); zero(dvu[nt]); }
#pragma unroll
  for (int jt = 0; jt < BT; ++jt) zero(dtacc[jt]);
  if (TC && HDP > HD) {
    lds_zero(s_kct + HD * LDC, (HDP - HD) * LDC);
    lds_zero(s_qut + HD * LDC, (HDP - HD) * LDC);
    for (int q = 0; q < NQ; ++q) {
      lds_zero(s_ubt[q] + HD * LDC, (HDP - HD) * LDC);
      lds_zero(s_gt[q] + HD * LDC, (HDP - HD) * LDC);
    }
  }

  PatchStage<T, TI, kCK, HD, 64> pi;
  PatchStage<T, T, kCK, HD, 64> pw;
  const int sq = wave & 1;                          // which of the two row blocks the workspace tile serves
  const int sblk = Ifirst + sq;
  const TI* isrc = wave == 0 ? kc : (wave == 1 ? qu : vc);
  const int64_t istride = wave == 0 ? a.kc.sl : (wave == 1 ? a.qu.sl : a.vc.sl);
// issue the global loads of the chunk that starts at key K0 (each wave its own tiles)
#define CASTLE_BQ_WANT_U(K0) (wave < 2 && sblk < a.s.nblk && (K0) / kNB < sblk)
#define CASTLE_BQ_WANT_G(K0) (wave >= 2 && sblk <= a.s.nblk - 2 && (K0) / kNB <= sblk)
#define CASTLE_BQ_LOAD(K0)                                                                          \
  do {                                                                                              \
    if (wave < 3) pi.load(lane, isrc, istride, (K0), L);                                            \
    if (CASTLE_BQ_WANT_U(K0)) pw.load(lane, usnap + usnap_off(sblk) * HD, HD, (K0), (int64_t)1 << 40); \
    if (CASTLE_BQ_WANT_G(K0)) pw.load(lane, gsnap + gsnap_off(sblk) * HD, HD, (K0), (int64_t)1 << 40); \
  } while (0)

  int kend = qb * QB + QB;
  if (kend > a.s.Lp) kend = a.s.Lp;
  CASTLE_BQ_LOAD(0);
  for (int k0 = 0; k0 < kend; k0 += kCK) {
    const int Kb = k0 / kNB;
    __syncthreads();
    // one wave per tile (wave 0: kc + ub[0], wave 1: qu + ub[1], wave 2: vc + g[0], wave 3: g[1]),
    // written from the registers the previous iteration filled; then the next chunk's loads go out
    if (wave < 3) {
      pi.store_rows(lane, wave == 0 ? s_kc : (wave == 1 ? s_qu : s_vc), LDK);
      if constexpr (TC) {
        if (wave < 2) pi.store_cols(lane, wave == 0 ? s_kct : s_qut, LDC);
      }
    }
    if (CASTLE_BQ_WANT_U(k0)) {
      pw.store_rows(lane, sq == 0 ? s_ub[0] : s_ub[1], LDK);
      if constexpr (TC) pw.store_cols(lane, sq == 0 ? s_ubt[0] : s_ubt[1], LDC);
    }
    if (CASTLE_BQ_WANT_G(k0)) {
      pw.store_rows(lane, sq == 0 ? s_g[0] : s_g[1], LDK);
      if constexpr (TC) pw.store_cols(lane, sq == 0 ? s_gt[0] : s_gt[1], LDC);
    }
    if (k0 + kCK < kend) CASTLE_BQ_LOAD(k0 + kCK);
    __syncthreads();
    const bool active = Kb <= Iw;

    // phase 0: gate tile A[k rows, j lanes] for this wave's 32 source rows
    acc_t aK;
    zero(aK);
    if (active) {
#pragma unroll
      for (int s = 0; s < KS; ++s) mma(aK, ld_nat<T>(s_qu, LDK, c, 16 * s + 8 * g), fku[s]);
#pragma unroll
      for (int r = 0; r < 16; ++r) aK[r] = fast_rcp(1.f + fast_exp2(aK[r]));
      if (k0 + 31 >= i0w) {   // chunk reaches the diagonal: keep j > k only
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (i <= k0 + acc_row(r, g)) aK[r] = 0.f;
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) s_a[acc_row(r, g) * LDA + jw + c] = (T)aK[r];
      if constexpr (TC) {
#pragma unroll
        for (int q = 0; q < 4; ++q) st4<T>(s_at + (jw + c) * LDC + 8 * q + 4 * g, pack4<T>(aK, q));
      }
    }
    __syncthreads();

    // phase 1: this lane's row is a query
    if (active && k0 <= i0w + 31) {
      acc_t sc, su, dp;
      zero(sc); zero(su); zero(dp);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        mma(sc, ld_nat<T>(s_kc, LDK, c, 16 * s + 8 * g), fqc[s]);
        if (Kb < Iw) mma(su, ld_nat<T>(s_ub[qw], LDK, c, 16 * s + 8 * g), fqc[s]);
        mma(dp, ld_nat<T>(s_vc, LDK, c, 16 * s + 8 * g), fdo[s]);
      }
#pragma unroll
      for (int s = 0; s < TS; ++s)
        if (s < nintra) mma(su, ld_nat<T>(s_a, LDA, c, cb + 16 * s + 8 * g), ft[s]);
      acc_t ds, dsu;
      const bool diag = k0 + 31 > i0w;   // chunk reaches the diagonal
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float sg = fast_rcp(1.f + fast_exp2(-su[r]));
        const float x = __builtin_fmaf(-su[r], sg, sc[r]);
        float p = fast_exp2(x - lse2);
        if (diag && k0 + acc_row(r, g) > i) p = 0.f;
        const float dsv = p * (dp[r] - dlt);
        const float y = su[r] * kLn2;                     // true Su
        const float t = __builtin_fmaf(-y, sg, y);
        const float sp = __builtin_fmaf(sg, t, sg);
        ds[r] = dsv;
        dsu[r] = -dsv * sp;
        s_dsu[acc_row(r, g) * LDA + jw + c] = (T)dsu[r];
      }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const frag<T> fds = chain<T>(ds, s2), fdsu = chain<T>(dsu, s2);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          mma(dqc[nt], ld_tr_chain<T>(s_kct, LDC, s_kc, LDK, 32 * nt + c, HD, 16 * s2, g), fds);
          if (Kb < Iw) mma(dqc[nt], ld_tr_chain<T>(s_ubt[qw], LDC, s_ub[qw], LDK, 32 * nt + c, HD, 16 * s2, g), fdsu);
        }
#pragma unroll
        for (int jt = 0; jt < BT; ++jt)
          if (32 * jt < lw + 32)
            mma(dtacc[jt], ld_tr_chain<T>(s_at, LDC, s_a, LDA, cb + 32 * jt + c, QB, 16 * s2, g), fdsu);
      }
    }
    __syncthreads();

    // phase 2: this lane's row is a lookahead source j; needs some key k < j
    if (active && k0 < i0w + 31) {
      acc_t dA;
      zero(dA);
#pragma unroll
      for (int s = 0; s < TS; ++s)
        if (s >= ifirst) mma(dA, ld_nat<T>(s_dsu, LDA, c, cb + 16 * s + 8 * g), ftt[s]);
      if (has_g) {
#pragma unroll
        for (int s = 0; s < KS; ++s) mma(dA, ld_nat<T>(s_g[qw], LDK, c, 16 * s + 8 * g), fvu[s]);
      }
      acc_t dz;
#pragma unroll
      for (int r = 0; r < 16; ++r) dz[r] = dA[r] * aK[r] * (1.f - aK[r]);
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const frag<T> fdz = chain<T>(dz, s2), fa = chain<T>(aK, s2);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          mma(dku[nt], ld_tr_chain<T>(s_qut, LDC, s_qu, LDK, 32 * nt + c, HD, 16 * s2, g), fdz);
          if (has_g) mma(dvu[nt], ld_tr_chain<T>(s_gt[qw], LDC, s_g[qw], LDK, 32 * nt + c, HD, 16 * s2, g), fa);
        }
      }
    }
  }

  // ---- epilogue: in-block terms dT = tril(dTacc):  dqc += dT Vu,  dvu += dT^T Qc -------------
  __syncthreads();
  Carver ce{castle_smem};
  T* e_vu[NQ]; T* e_qc[NQ]; T* e_vut[NQ]; T* e_qct[NQ]; T* e_dt[NQ];
  for (int q = 0; q < NQ; ++q) e_vu[q] = ce.take<T>(kNB * LDK);
  for (int q = 0; q < NQ; ++q) e_qc[q] = ce.take<T>(kNB * LDK);
  for (int q = 0; q < NQ; ++q) { e_vut[q] = e_vu[q]; e_qct[q] = e_qc[q]; }
  if constexpr (TC) {
    for (int q = 0; q < NQ; ++q) e_vut[q] = ce.take<T>(HDP * LDV);
    for (int q = 0; q < NQ; ++q) e_qct[q] = ce.take<T>(HDP * LDQ);
  }
  for (int q = 0; q < NQ; ++q) e_dt[q] = ce.take<T>(kNB * LDT);
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int64_t r0 = (int64_t)(Ifirst + q) * kNB;
    RowStage<T, TI, kNB, HD> st;
    st.load(vu, a.vu.sl, r0, L); st.store(e_vu[q], LDK);
    st.load(qc, a.qc.sl, r0, L); st.store_scaled(e_qc[q], LDK, c1);
    if constexpr (TC) {
      if (HDP > HD) {
        lds_zero(e_vut[q] + HD * LDV, (HDP - HD) * LDV);
        lds_zero(e_qct[q] + HD * LDQ, (HDP - HD) * LDQ);
      }
      ColStage<T, TI, kNB, HD> ct;
      ct.load(vu, a.vu.sl, r0, L); ct.store(e_vut[q], LDV);
      ct.load(qc, a.qc.sl, r0, L); ct.store(e_qct[q], LDQ, c1);
    }
  }
  // dT^T[j rows, i lanes] masked to j <= i, shared as e_dt[j][i] for the source-side product
#pragma unroll
  for (int jt = 0; jt < BT; ++jt) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int jl = 32 * jt + acc_row(r, g);
      if (jl > lw + c) dtacc[jt][r] = 0.f;
      e_dt[qw][jl * LDT + lw + c] = (T)dtacc[jt][r];
    }
  }
  __syncthreads();
#pragma unroll
  for (int jt = 0; jt < BT; ++jt) {
    if (32 * jt >= lw + 32) continue;
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const frag<T> fdt = chain<T>(dtacc[jt], s2);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        mma(dqc[nt], ld_tr_chain<T>(e_vut[qw], LDV, e_vu[qw], LDK, 32 * nt + c, HD, 32 * jt + 16 * s2, g), fdt);
    }
  }
#pragma unroll
  for (int s = 0; s < TS; ++s) {
    if (s < ifirst) continue;
    const frag<T> fdt = ld_nat<T>(e_dt[qw], LDT, lw + c, 16 * s + 8 * g);   // (source j, queries i)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      mma(dvu[nt], ld_tr_nat<T>(e_qct[qw], LDQ, e_qc[qw], LDK, 32 * nt + c, HD, 16 * s, g), fdt);
  }
  if (i < L) {
    store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dqc, b, h) + (int64_t)i * a.dqc.sl, dqc, c0, g);
    store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dku, b, h) + (int64_t)i * a.dku.sl, dku, c0 * kLn2, g);
    store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dvu, b, h) + (int64_t)i * a.dvu.sl, dvu, kLn2, g);
  }
}

// ---------------------------------------------------------------------------
template <typename T, typename TI, int HD> static int launch_bwd_t(const BwdArgs& a, hipStream_t stream) {
  const int BH = a.s.B * a.s.H;
  constexpr int key_lds = bwd_key_lds_bytes<T, HD>(), query_lds = bwd_query_lds_bytes<T, HD>();
  if (key_lds > kMaxLds || query_lds > kMaxLds) return -2;
  static bool configured = false;   // raising the dynamic-LDS limit is idempotent, so a race is harmless
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_key_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, key_lds) != hipSuccess) return -3;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_query_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, query_lds) != hipSuccess) return -3;
    configured = true;
  }
  constexpr int RPB = kThreads / (HD / elem_traits<T>::vec16);
  {
    ProfScope ps(kSlotDelta, stream);
    hipLaunchKernelGGL((delta_kernel<TI, HD>), dim3((a.s.Lp + RPB - 1) / RPB, BH), dim3(kThreads), 0, stream, a);
  }
  {
    ProfScope ps(kSlotBwdKey, stream);
    hipLaunchKernelGGL((bwd_key_kernel<T, TI, HD>), dim3(a.s.Lp / 128 * BH), dim3(kThreads), key_lds, stream, a);
  }
  {
    ProfScope ps(kSlotBwdQuery, stream);
    hipLaunchKernelGGL((bwd_query_kernel<T, TI, HD>), dim3(a.s.Lp / 128 * BH), dim3(kThreads), query_lds, stream, a);
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <typename T, typename TI> static int launch_bwd_d(const BwdArgs& a, hipStream_t stream) {
  switch (a.s.d) {
    case 16: return launch_bwd_t<T, TI, 16>(a, stream);
    case 32: return launch_bwd_t<T, TI, 32>(a, stream);
    case 64: return launch_bwd_t<T, TI, 64>(a, stream);
    default: return -2;   // d = 128: the register budget of the key-stationary kernel is exceeded
  }
}

// bf16 tensors use fp16 MFMA operands unless bf16_operands is set (must match the forward pass,
// whose workspace holds operands in the compute type)
int launch_bwd(const BwdArgs& a, int dtype, bool bf16_operands, hipStream_t stream) {
  switch (dtype) {
    case 0: return launch_bwd_d<float, float>(a, stream);
    case 1: return bf16_operands ? launch_bwd_d<bf16_t, bf16_t>(a, stream) : launch_bwd_d<fp16_t, bf16_t>(a, stream);
    case 2: return launch_bwd_d<fp16_t, fp16_t>(a, stream);
    default: return -1;
  }
}

}  // namespace castle
