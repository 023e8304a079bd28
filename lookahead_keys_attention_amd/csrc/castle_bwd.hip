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
// Those two are the single-role kernels (fp32 tensors; 16-bit at d = 128 without room for score
// tiles).  16-bit tensors otherwise run workgroups of 512 threads in two wave roles that share a
// SIMD pairwise, and hand dS / dSu from the key side to the query side as 32 x 32 tiles in HBM:
//   bwd_key2_kernel   (d <= 64) score waves + gradient waves, one launch
//   bwd_keyw1_kernel, bwd_keyw2_kernel  (d = 128) the same split over two launches
//   bwd_query2_kernel source-row waves + query-row waves; one launch up to d = 64, two at d = 128
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
// Writes one gradient row held as accumulator tiles [n rows, this lane's row].  rope_pos >= 0: the
// operand was rotated by that position before use, so its gradient is rotated back first.
// The NT tiles are columns 32 nt0 .. 32 (nt0 + NT) - 1 of the row.
template <typename T, int HD, int NT>   // T: element type of the destination tensor
__device__ __forceinline__ void store_rows(T* dst_row, acc_t (&acc)[NT], float mul, int g, int rope_pos = -1, int nt0 = 0) {
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    if (rope_pos >= 0) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = 32 * (nt0 + nt) + 8 * q + 4 * g;
        if (n < HD) {
          CASTLE_ROPE_PAIR(acc[nt][4 * q], acc[nt][4 * q + 1], (float)rope_pos, n / 2, HD, true);
          CASTLE_ROPE_PAIR(acc[nt][4 * q + 2], acc[nt][4 * q + 3], (float)rope_pos, n / 2 + 1, HD, true);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nt][r] *= mul;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = 32 * (nt0 + nt) + 8 * q + 4 * g;
      if (n < HD) st4<T>(dst_row + n, pack4<T>(acc[nt], q));
    }
  }
}

// ---------------------------------------------------------------------------
// delta = rowsum(dO * O); also leaves dO in the compute type, padded to Lp rows, for the other kernels
template <typename T, typename TI, int HD>
__global__ __launch_bounds__(kThreads) void delta_kernel(BwdArgs a) {
  constexpr int V = elem_traits<TI>::vec16;
  constexpr int LPR = HD / V;
  constexpr int RPB = kThreads / LPR;
  typedef vec<TI, V> vt;
  const int bh = blockIdx.y, b = bh / a.s.H, h = bh % a.s.H;
  const int grp = threadIdx.x / LPR, sub = threadIdx.x % LPR;
  const int64_t i = (int64_t)blockIdx.x * RPB + grp;
  // 16-bit operands: the whole backward runs on dO * gs, gs the power of two that puts max|dO| into
  // [16, 32), so that neither tiny nor huge upstream gradients leave the fp16 range on their way
  // through dS, dSu, dZ and the reverse state; the gradient stores multiply by 1 / gs
  float gs = 1.f;
  if constexpr (sizeof(T) == 2) gs = pow2_placing(amax_from_partials(a.amax_part), 4);
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
    a.bhdr->grad_scale = gs;
    a.bhdr->grad_unscale = 1.f / gs;
  }
  if (i >= a.s.Lp) return;
  float acc = 0.f;
  vt d;
#pragma unroll
  for (int e = 0; e < V; ++e) d[e] = (TI)0.f;
  if (i < a.s.L) {
    vt o = *reinterpret_cast<const vt*>(head_ptr<TI>(a.out, b, h) + i * a.out.sl + sub * V);
    d = *reinterpret_cast<const vt*>(head_ptr<TI>(a.dout, b, h) + i * a.dout.sl + sub * V);
#pragma unroll
    for (int e = 0; e < V; ++e) acc = __builtin_fmaf((float)o[e], (float)d[e], acc);
  }
  vec<float, V> ds = __builtin_convertvector(d, vec<float, V>);
#pragma unroll
  for (int e = 0; e < V; ++e) ds[e] *= gs;
  *reinterpret_cast<vec<T, V>*>(reinterpret_cast<T*>(a.dout_p) + ((int64_t)bh * a.s.Lp + i) * HD + sub * V) = __builtin_convertvector(ds, vec<T, V>);
#pragma unroll
  for (int o = 1; o < LPR; o <<= 1) acc += __shfl_xor(acc, o);
  if (sub == 0) a.delta[(int64_t)bh * a.s.Lp + i] = acc * gs;
}

// ---------------------------------------------------------------------------
template <typename T, int HD> constexpr int bwd_key_lds_bytes() {
  int b = 0;
  b += 3 * a16((int)sizeof(T) * kNB * lds_ld<T>(HD));           // qc, do, ku
  b += a16((int)sizeof(T) * kNB * lds_ld_chain<T>(HD));         // vu
  b += a16((int)sizeof(T) * kNB * lds_ld_chain<T>(kNB));        // T
  b += 2 * a16(4 * kNB);                                        // lse, delta
  if (HD > 64) b += 2 * a16((int)sizeof(T) * 128 * lds_ld<T>(HD));   // kc, vc rows of the workgroup (d = 128: not in registers)
  return b;
}

// PART selects the outputs of a launch: 0 = all (d <= 64); 1 = dVc, dKc; 2 = dQu and the reverse
// state (gsnap).  At d = 128 the four accumulator sets do not fit the register file together, so
// the kernel runs once with PART 1 and once with PART 2.  This is the kernel of fp32 tensors, and
// of 16-bit tensors at d = 128 when there is no room for the dS / dSu tiles (otherwise the two-role
// kernels below run).
template <typename T, typename TI, int HD, int PART>
__global__ __launch_bounds__(kThreads, 1) void bwd_key_kernel(BwdArgs a) {
  constexpr bool DO_KV = PART != 2, DO_QG = PART != 1;
  constexpr int KS = HD / 16;
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr int NT = HDP / 32;
  constexpr int BT = kNB / 32;   // 32-row sub-tiles per block
  constexpr int LDK = lds_ld<T>(HD), LDU = lds_ld_chain<T>(HD), LDT = lds_ld_chain<T>(kNB);

  Carver cv{castle_smem};
  T* s_qc = cv.take<T>(kNB * LDK);
  T* s_do = cv.take<T>(kNB * LDK);
  T* s_ku = cv.take<T>(kNB * LDK);
  T* s_vu = cv.take<T>(kNB * LDU);
  T* s_t = cv.take<T>(kNB * LDT);
  float* s_lse = cv.take<float>(kNB);
  float* s_delta = cv.take<float>(kNB);
  // At d = 128 the score chain takes the kc / vc rows of the workgroup's keys from LDS instead of
  // holding them in registers: that is what leaves room for the register prefetch of the next block.
  constexpr bool KV_LDS = HD > 64;
  T* s_kcw = KV_LDS ? cv.take<T>(128 * LDK) : nullptr;
  T* s_vcw = KV_LDS ? cv.take<T>(128 * LDK) : nullptr;

  int kb, bh;   // key group 0 meets every query block: rank order = kb
  work_item(a.s.B * a.s.H, kb, bh);
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const int L = a.s.L;
  const float c0 = a.s.scale, c1 = a.s.scale * kLog2e;
  const float su_mul = a.ws.hdr->su_mul, gun = a.bhdr->grad_unscale;
  const int kw0 = kb * 128 + 32 * wave;
  const int k = kw0 + c;
  const int Iw = kw0 / kNB;
  const T* qc = prep_ptr<T>(a.ws.qc_p, bh, a.s.Lp, HD);
  const T* kc = prep_ptr<T>(a.ws.kc_p, bh, a.s.Lp, HD);
  const T* vc = prep_ptr<T>(a.ws.vc_p, bh, a.s.Lp, HD);
  const T* qu = prep_ptr<T>(a.ws.qu_p, bh, a.s.Lp, HD);
  const T* ku = prep_ptr<T>(a.ws.ku_p, bh, a.s.Lp, HD);
  const T* vu = prep_ptr<T>(a.ws.vu_p, bh, a.s.Lp, HD);
  const T* dout = prep_ptr<T>(a.dout_p, bh, a.s.Lp, HD);
  const T* tb = reinterpret_cast<const T*>(a.ws.t_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* usnap = reinterpret_cast<const T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  T* gsnap = reinterpret_cast<T*>(a.gsnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  const float* lse = a.ws.lse + (int64_t)bh * a.s.Lp;
  const float* delta = a.delta + (int64_t)bh * a.s.Lp;

  constexpr int NKV = KV_LDS ? 1 : KS;
  frag<T> fkc[NKV], fvc[NKV], fqu[KS], fub[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) fqu[s] = ldg_nat_scaled<T, T>(qu, HD, k, 16 * s + 8 * g, true, -c1);
#pragma unroll
  for (int s = 0; s < KS; ++s) fub[s] = zero_frag<T>();
  if constexpr (KV_LDS) {   // visible after the first barrier of the block loop
    RowStage<T, T, 128, HD> st;
    st.load_flat(kc + (int64_t)kb * 128 * HD); st.store(s_kcw, LDK);
    st.load_flat(vc + (int64_t)kb * 128 * HD); st.store(s_vcw, LDK);
  } else {
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      fkc[s] = ldg_nat<T>(kc, HD, k, 16 * s + 8 * g, true);
      fvc[s] = ldg_nat<T>(vc, HD, k, 16 * s + 8 * g, true);
    }
  }
  acc_t dvc[NT], dkc[NT], dqu[NT], G[NT];   // [n rows, k lanes]
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) { zero(dvc[nt]); zero(dkc[nt]); zero(dqu[nt]); zero(G[nt]); }

  // every thread carries its 16-byte pieces of the five tiles of the next block
  RowStage<T, T, kNB, HD> pqc, pdo, pku, pvu;
  RowStage<T, T, kNB, kNB> ptb;
#define CASTLE_BK_LOAD(I_)                                   \
  do {                                                       \
    const int64_t r_ = (int64_t)(I_) * kNB;                  \
    pqc.load_flat(qc + r_ * HD);                            \
    pdo.load_flat(dout + r_ * HD);                          \
    pku.load_flat(ku + r_ * HD);                            \
    pvu.load_flat(vu + r_ * HD);                            \
    ptb.load(tb, kNB, r_, (int64_t)1 << 40);                 \
  } while (0)

  const int I0 = (kb * 128) / kNB;
  constexpr bool PF = true;   // every variant keeps the next block in flight in registers
  if (PF) CASTLE_BK_LOAD(a.s.nblk - 1);
  for (int I = a.s.nblk - 1; I >= I0; --I) {
    const bool active = I >= Iw;
    // reverse state as of block I; the tile-consuming query kernel only reads those behind a pair
    // of blocks (odd I), the recomputing one all of them
    if (DO_QG && active && I <= a.s.nblk - 2 && (a.ds_mat == nullptr || (I & 1))) {
      store_snap_tile<T, HD, NT>(gsnap + (gsnap_off(I) + kw0) * HD, G, c, g);
    }
    if (I > Iw) {
#pragma unroll
      for (int s = 0; s < KS; ++s) fub[s] = ldg_snap_nat<T>(usnap + (usnap_off(I) + kw0) * HD, c, 16 * s + 8 * g);
    }
    __syncthreads();
    const int64_t r0 = (int64_t)I * kNB;
    if (!PF) CASTLE_BK_LOAD(I);
    pqc.store(s_qc, LDK);
    pdo.store(s_do, LDK);
    pku.store(s_ku, LDK);
    pvu.store_halves(s_vu, LDU);
    ptb.store_halves(s_t, LDT);
    if (PF && I > I0) CASTLE_BK_LOAD(I - 1);   // in flight while this block is processed
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
      {
        frag<T> oku[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) oku[s] = ld_nat<T>(s_ku, LDK, 32 * jt + c, 16 * s + 8 * g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS; ++s) mma(aT[jt], oku[s], fqu[s]);
      }
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
      if constexpr (DO_QG) {
        frag<T> ovu[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) ovu[s] = ld_chain<T>(s_vu, LDU, 32 * jt + c, 16 * s, g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS; ++s) mma(dA[jt], ovu[s], chain<T>(G[s / 2], s % 2));
      }
    }
    // (c) query sub-tiles of the block
#pragma unroll
    for (int it = 0; it < BT; ++it) {
      const int i0 = I * kNB + 32 * it;
      if (i0 + 31 < kw0) continue;   // every query precedes every key of this wave
      acc_t sc, su, dp;
      zero(sc); zero(su); zero(dp);
      {
        frag<T> oq[KS], od[KS], ot[BT][2];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          oq[s] = ld_nat<T>(s_qc, LDK, 32 * it + c, 16 * s + 8 * g);
          od[s] = ld_nat<T>(s_do, LDK, 32 * it + c, 16 * s + 8 * g);
        }
#pragma unroll
        for (int jt = 0; jt < BT; ++jt)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2)
            if (jt <= it) ot[jt][s2] = ld_chain<T>(s_t, LDT, 32 * it + c, 32 * jt + 16 * s2, g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          if constexpr (KV_LDS) {
            mma(sc, oq[s], ld_nat<T>(s_kcw, LDK, 32 * wave + c, 16 * s + 8 * g));
            mma(dp, od[s], ld_nat<T>(s_vcw, LDK, 32 * wave + c, 16 * s + 8 * g));
          } else {
            mma(sc, oq[s], fkc[s]);
            mma(dp, od[s], fvc[s]);
          }
        }
        if (I > Iw) {
#pragma unroll
          for (int s = 0; s < KS; ++s) mma(su, oq[s], fub[s]);
        }
#pragma unroll
        for (int jt = 0; jt < BT; ++jt)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2)
            if (jt <= it) mma(su, ot[jt][s2], fa[jt][s2]);
      }
      acc_t ds, dsu;
      const bool diag = i0 < kw0 + 31;   // tile touches the diagonal
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int il = 32 * it + acc_row(r, g);
        const float sut = su[r] * su_mul;                 // log2(e) * Su
        const float sg = fast_rcp(1.f + fast_exp2(-sut));
        const float x = __builtin_fmaf(-sut, sg, sc[r]);
        float p = fast_exp2(x - s_lse[il]);
        if (diag && I * kNB + il < k) p = 0.f;
        const float dsv = p * (dp[r] - s_delta[il]);
        const float y = sut * kLn2;                       // true Su
        const float t = __builtin_fmaf(-y, sg, y);        // y (1 - sigmoid)
        const float sp = __builtin_fmaf(sg, t, sg);       // silu'(y)
        sc[r] = p;
        ds[r] = dsv;
        dsu[r] = -dsv * sp * su_mul;                      // gradient of the product built from vu * vu_scale
      }
      {
        frag<T> odt[2][NT], oqt[2][NT], ott[2][BT];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const int ic = 32 * it + 16 * s2;
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            if constexpr (DO_KV) odt[s2][nt] = ld_free<T, true>(s_do, LDK, 32 * nt, HD, ic, c, g);
            oqt[s2][nt] = ld_free<T, true>(s_qc, LDK, 32 * nt, HD, ic, c, g);
          }
          if constexpr (DO_QG) {
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
              if (jt <= it) ott[s2][jt] = ld_free<T, true>(s_t, LDT, 32 * jt, kNB, ic, c, g);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const frag<T> fp = chain<T>(sc, s2), fds = chain<T>(ds, s2), fdsu = chain<T>(dsu, s2);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            if constexpr (DO_KV) {
              mma(dvc[nt], odt[s2][nt], fp);
              mma(dkc[nt], oqt[s2][nt], fds);
            }
            if constexpr (DO_QG) mma(G[nt], oqt[s2][nt], fdsu);
          }
          if constexpr (DO_QG) {
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
              if (jt <= it) mma(dA[jt], ott[s2][jt], fdsu);
          }
        }
      }
    }
    // (d) dZ^T = dA^T * A (1 - A)  ->  dQu
#pragma unroll
    for (int jt = 0; jt < (DO_QG ? BT : 0); ++jt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) dA[jt][r] *= aT[jt][r] * (1.f - aT[jt][r]);
      {
        frag<T> okt[2][NT];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) okt[s2][nt] = ld_free<T, true>(s_ku, LDK, 32 * nt, HD, 32 * jt + 16 * s2, c, g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const frag<T> fdz = chain<T>(dA[jt], s2);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) mma(dqu[nt], okt[s2][nt], fdz);
        }
      }
    }
  }
#undef CASTLE_BK_LOAD
  if (k < L) {
    if constexpr (DO_KV) {
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dkc, b, h) + (int64_t)k * a.dkc.sl, dkc, kLn2 * gun, g, a.s.rotary ? k : -1);
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dvc, b, h) + (int64_t)k * a.dvc.sl, dvc, gun, g);
    }
    if constexpr (DO_QG) store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dqu, b, h) + (int64_t)k * a.dqu.sl, dqu, c0 * kLn2 * gun, g, a.s.rotary ? k : -1);
  }
}

// ---------------------------------------------------------------------------
// Key-stationary backward with two wave roles (16-bit compute types, d <= 64): 512 threads,
// waves 0-3 "score" waves, waves 4-7 "gradient" waves; pair (w, w + 4) owns keys
// kb*128 + 32 w .. + 31 and is expected to share a SIMD, so the element-wise chain of one role
// overlaps the MFMAs of the other.  Per 64-query block I (swept from the last one down):
//   score wave:    per 32-query sub-tile the scores, P, dS, dSu, handed over through LDS as
//                  [key][query] tiles; then the gate A of the NEXT block (-> A(1-A) for the partner)
//   gradient wave: dZ and dQu of the PREVIOUS block, reverse state G (snapshot, G Vu^T), then
//                  dVc, dKc, G, dA from the handed tiles; it also stores the dS / dSu tiles for
//                  the query-stationary kernel
// The gradient wave runs one sub-tile behind the score wave; four barriers per block, and in each
// of the three compute slots between them both roles have about the same amount of work.
// The Ku tile and the A(1-A) tiles are double buffered because they outlive their block.
template <typename T, int HD> constexpr int bwd_key2_lds_bytes() {
  int b = bwd_key_lds_bytes<T, HD>();
  b += a16((int)sizeof(T) * kNB * lds_ld<T>(HD));           // second Ku tile
  b += 4 * 3 * a16((int)sizeof(T) * 32 * lds_ld<T>(kNB));   // P, dS, dSu per wave pair
  b += 2 * 4 * a16((int)sizeof(T) * 32 * lds_ld<T>(kNB));   // A (1 - A) per wave pair, two blocks
  return b;
}

template <typename T, typename TI, int HD>
__global__ __launch_bounds__(2 * kThreads, 1) void bwd_key2_kernel(BwdArgs a) {
  static_assert(sizeof(T) == 2 && HD <= 64, "two-role kernel: 16-bit operands, d <= 64");
  constexpr int KS = HD / 16;
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr int NT = HDP / 32;
  constexpr int BT = kNB / 32;
  constexpr int LDK = lds_ld<T>(HD), LDU = lds_ld_chain<T>(HD), LDT = lds_ld_chain<T>(kNB);
  constexpr int LDX = lds_ld<T>(kNB);

  Carver cv{castle_smem};
  T* s_qc = cv.take<T>(kNB * LDK);
  T* s_do = cv.take<T>(kNB * LDK);
  T* s_ku0 = cv.take<T>(kNB * LDK);
  T* s_ku1 = cv.take<T>(kNB * LDK);
  T* s_vu = cv.take<T>(kNB * LDU);
  T* s_t = cv.take<T>(kNB * LDT);
  float* s_lse = cv.take<float>(kNB);
  float* s_delta = cv.take<float>(kNB);
  T* s_x = cv.take<T>(4 * 3 * 32 * LDX);
  T* s_w = cv.take<T>(2 * 4 * 32 * LDX);

  int kb, bh;
  work_item(a.s.B * a.s.H, kb, bh);
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const bool scorer = wave < 4;
  const int pw = wave & 3;
  const int L = a.s.L;
  const float c0 = a.s.scale, c1 = a.s.scale * kLog2e;
  const float su_mul = a.ws.hdr->su_mul, gun = a.bhdr->grad_unscale;
  const int kw0 = kb * 128 + 32 * pw;
  const int k = kw0 + c;
  const int Iw = kw0 / kNB;
  const int I0 = (kb * 128) / kNB;
  const int Ilast = a.s.nblk - 1;
  T* x_p = s_x + pw * 3 * 32 * LDX;   // [key][query of the block]
  T* x_ds = x_p + 32 * LDX;
  T* x_dsu = x_ds + 32 * LDX;
  T* x_w = s_w + pw * 32 * LDX;       // [key][source of the block], + 4*32*LDX for odd blocks

  const T* qc = prep_ptr<T>(a.ws.qc_p, bh, a.s.Lp, HD);
  const T* ku = prep_ptr<T>(a.ws.ku_p, bh, a.s.Lp, HD);
  const T* vu = prep_ptr<T>(a.ws.vu_p, bh, a.s.Lp, HD);
  const T* dout = prep_ptr<T>(a.dout_p, bh, a.s.Lp, HD);
  const T* tb = reinterpret_cast<const T*>(a.ws.t_blk) + (int64_t)bh * a.s.Lp * kNB;
  // The score waves (threads 0..255) stage the five tiles of a block: the loads of block I - 1 are
  // issued right after the tiles of block I have been written.  Ku (needed first, by the gate of
  // the next block) goes to its other buffer one slot later, the rest when block I is done.
  // The gradient waves keep out of it: their global stores would sit in front of such loads in
  // the in-order memory counter.
#define CASTLE_BK2_STAGE_DECL                 \
  RowStage<T, T, kNB, HD> pku, pqc, pdo, pvu; \
  RowStage<T, T, kNB, kNB> ptb;               \
  float plse = 0.f, pdelta = 0.f
#define CASTLE_BK2_STAGE_LOAD(I_)                            \
  do {                                                       \
    const int64_t r_ = (int64_t)(I_) * kNB;                  \
    pku.load_flat(ku + r_ * HD);                             \
    pqc.load_flat(qc + r_ * HD);                             \
    pdo.load_flat(dout + r_ * HD);                           \
    pvu.load_flat(vu + r_ * HD);                             \
    ptb.load_flat(tb + r_ * kNB);                            \
    if (threadIdx.x < kNB) {                                 \
      const int64_t i_ = r_ + threadIdx.x;                   \
      plse = i_ < L ? lse[i_] : INFINITY;                    \
      pdelta = i_ < L ? delta[i_] : 0.f;                     \
    }                                                        \
  } while (0)
#define CASTLE_BK2_STAGE_STORE()                             \
  do {                                                       \
    pqc.store(s_qc, LDK);                         \
    pdo.store(s_do, LDK);                                    \
    pvu.store_halves(s_vu, LDU);                             \
    ptb.store_halves(s_t, LDT);                              \
    if (threadIdx.x < kNB) {                                 \
      s_lse[threadIdx.x] = -plse * kLog2e;                   \
      s_delta[threadIdx.x] = -pdelta;                        \
    }                                                        \
  } while (0)
#define CASTLE_BK2_KU(I_) (((I_) & 1) ? s_ku1 : s_ku0)
#define CASTLE_BK2_W(I_) (x_w + ((I_) & 1) * 4 * 32 * LDX)

  if (scorer) {
    const T* kc = prep_ptr<T>(a.ws.kc_p, bh, a.s.Lp, HD);
    const T* vc = prep_ptr<T>(a.ws.vc_p, bh, a.s.Lp, HD);
    const T* qu = prep_ptr<T>(a.ws.qu_p, bh, a.s.Lp, HD);
    const T* usnap = reinterpret_cast<const T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
    const float* lse = a.ws.lse + (int64_t)bh * a.s.Lp;
    const float* delta = a.delta + (int64_t)bh * a.s.Lp;

    frag<T> fkc[KS], fvc[KS], fqu[KS], fub[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      fkc[s] = ldg_nat<T>(kc, HD, k, 16 * s + 8 * g, true);
      fvc[s] = ldg_nat<T>(vc, HD, k, 16 * s + 8 * g, true);
      fqu[s] = ldg_nat_scaled<T, T>(qu, HD, k, 16 * s + 8 * g, true, -c1);
      fub[s] = zero_frag<T>();
    }
    CASTLE_BK2_STAGE_DECL;
    frag<T> fa[BT][2];
    // gate tiles A^T[j rows, k lanes] of source block J: operand fragments for the score tiles of
    // that block and A (1 - A) for the partner wave
#define CASTLE_BK2_GATE(J_)                                                                          \
  do {                                                                                               \
    const T* ku_tile_ = CASTLE_BK2_KU(J_);                                                           \
    T* w_tile_ = CASTLE_BK2_W(J_);                                                                   \
    _Pragma("unroll") for (int jt = 0; jt < BT; ++jt) {                                              \
      acc_t aT;                                                                                      \
      zero(aT);                                                                                      \
      {                                                                                              \
        frag<T> oku[KS];                                                                             \
        _Pragma("unroll") for (int s = 0; s < KS; ++s)                                               \
          oku[s] = ld_nat<T>(ku_tile_, LDK, 32 * jt + c, 16 * s + 8 * g);                            \
        __builtin_amdgcn_sched_barrier(0);                                                           \
        _Pragma("unroll") for (int s = 0; s < KS; ++s) mma(aT, oku[s], fqu[s]);                      \
      }                                                                                              \
      const int j0 = (J_) * kNB + 32 * jt;                                                           \
      _Pragma("unroll") for (int r = 0; r < 16; ++r) aT[r] = fast_rcp(1.f + fast_exp2(aT[r]));       \
      if (j0 <= kw0 + 31) { /* tile touches the diagonal: keep j > k only */                         \
        _Pragma("unroll") for (int r = 0; r < 16; ++r)                                               \
          if (j0 + acc_row(r, g) <= k) aT[r] = 0.f;                                                  \
      }                                                                                              \
      fa[jt][0] = chain<T>(aT, 0);                                                                   \
      fa[jt][1] = chain<T>(aT, 1);                                                                   \
      _Pragma("unroll") for (int r = 0; r < 16; ++r) aT[r] = __builtin_fmaf(-aT[r], aT[r], aT[r]);         \
      _Pragma("unroll") for (int q = 0; q < 4; ++q)                                                  \
        st4<T>(w_tile_ + c * LDX + 32 * jt + 8 * q + 4 * g, pack4<T>(aT, q));                        \
    }                                                                                                \
  } while (0)

    CASTLE_BK2_STAGE_LOAD(Ilast);
    if (Ilast > Iw) {
#pragma unroll
      for (int s = 0; s < KS; ++s) fub[s] = ldg_snap_nat<T>(usnap + (usnap_off(Ilast) + kw0) * HD, c, 16 * s + 8 * g);
    }
    pku.store(CASTLE_BK2_KU(Ilast), LDK);
    __syncthreads();   // 0: first Ku tile staged
    if (Ilast >= Iw) CASTLE_BK2_GATE(Ilast);
    for (int I = Ilast; I >= I0; --I) {
      const bool active = I >= Iw;
      const bool inter = I > Iw;   // lookahead state from earlier blocks exists
      CASTLE_BK2_STAGE_STORE();
      // The staged pieces were the oldest loads in flight, so the lookahead state requested after
      // them has arrived too; pin that here, or the wait for it would land behind the loads of
      // the next block, which are issued below.
#pragma unroll
      for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(fub[s]));
      __syncthreads();   // 1: tiles staged
      if (I > I0) CASTLE_BK2_STAGE_LOAD(I - 1);   // in flight for the whole block
#pragma unroll
      for (int it = 0; it < BT; ++it) {
        if (it == 1 && I > I0) pku.store(CASTLE_BK2_KU(I - 1), LDK);
        const int i0 = I * kNB + 32 * it;
        if (active && i0 + 31 >= kw0) {   // else every query precedes every key of this wave
          acc_t sc, su, dp;   // sc starts from -lse, dp from -delta of its row
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const vec<float, 4> nl = *reinterpret_cast<const vec<float, 4>*>(s_lse + 32 * it + 8 * q + 4 * g);
            const vec<float, 4> nd = *reinterpret_cast<const vec<float, 4>*>(s_delta + 32 * it + 8 * q + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              sc[4 * q + e] = nl[e];
              dp[4 * q + e] = nd[e];
              su[4 * q + e] = 0.f;
            }
          }
          {
            frag<T> oq[KS], od[KS], ot[BT][2];
#pragma unroll
            for (int s = 0; s < KS; ++s) {
              oq[s] = ld_nat<T>(s_qc, LDK, 32 * it + c, 16 * s + 8 * g);
              od[s] = ld_nat<T>(s_do, LDK, 32 * it + c, 16 * s + 8 * g);
            }
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
#pragma unroll
              for (int s2 = 0; s2 < 2; ++s2)
                if (jt <= it) ot[jt][s2] = ld_chain<T>(s_t, LDT, 32 * it + c, 32 * jt + 16 * s2, g);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < KS; ++s) {
              mma(sc, oq[s], fkc[s]);
              mma(dp, od[s], fvc[s]);
            }
            if (inter) {
#pragma unroll
              for (int s = 0; s < KS; ++s) mma(su, oq[s], fub[s]);
            }
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
#pragma unroll
              for (int s2 = 0; s2 < 2; ++s2)
                if (jt <= it) mma(su, ot[jt][s2], fa[jt][s2]);
          }
          acc_t ds, dsu;
          if (i0 < kw0 + 31) {   // tile touches the diagonal: queries before the key see nothing
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if (i0 + acc_row(r, g) < k) sc[r] = -INFINITY;
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float sut = su[r] * su_mul;                 // log2(e) * Su
            const float sg = fast_rcp(1.f + fast_exp2(-sut));
            const float p = fast_exp2(__builtin_fmaf(-sut, sg, sc[r]));   // sc carries -lse
            const float dsv = p * dp[r];                      // dp carries -delta
            const float y = sut * kLn2;                       // true Su
            const float t = __builtin_fmaf(-y, sg, y);        // y (1 - sigmoid)
            const float sp = __builtin_fmaf(sg, t, sg);       // silu'(y)
            sc[r] = p;
            ds[r] = dsv;
            dsu[r] = -dsv * sp * su_mul;                      // gradient of the product built from vu * vu_scale
          }
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int o = c * LDX + 32 * it + 8 * q + 4 * g;
            st4<T>(x_p + o, pack4<T>(sc, q));
            st4<T>(x_ds + o, pack4<T>(ds, q));
            st4<T>(x_dsu + o, pack4<T>(dsu, q));
          }
        }
        __syncthreads();   // 2, 3: sub-tile handed over
      }
      if (I > I0) {
        if (I - 1 > Iw) {   // lookahead state as of the next block: in flight behind the gate
#pragma unroll
          for (int s = 0; s < KS; ++s) fub[s] = ldg_snap_nat<T>(usnap + (usnap_off(I - 1) + kw0) * HD, c, 16 * s + 8 * g);
        }
        if (I - 1 >= Iw) CASTLE_BK2_GATE(I - 1);   // while the gradient waves finish block I
      }
      __syncthreads();   // 4: tiles free
    }
#undef CASTLE_BK2_GATE
  } else {
    T* gsnap = reinterpret_cast<T*>(a.gsnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
    T* ds_mat = reinterpret_cast<T*>(a.ds_mat) + (int64_t)bh * a.s.Lp * a.s.Lp;
    T* dsu_mat = reinterpret_cast<T*>(a.dsu_mat) + (int64_t)bh * a.s.Lp * a.s.Lp;
    acc_t dvc[NT], dkc[NT], dqu[NT], G[NT];   // [n rows, k lanes]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) { zero(dvc[nt]); zero(dkc[nt]); zero(dqu[nt]); zero(G[nt]); }
    acc_t dA[BT];   // dA^T[j rows, k lanes] of the block in flight
#pragma unroll
    for (int jt = 0; jt < BT; ++jt) zero(dA[jt]);
    // dZ^T = dA^T * A (1 - A)  ->  dQu, for source block J (its Ku tile and A(1-A) are still there)
#define CASTLE_BK2_DQU(J_)                                                                           \
  do {                                                                                               \
    const T* ku_tile_ = CASTLE_BK2_KU(J_);                                                           \
    const T* w_tile_ = CASTLE_BK2_W(J_);                                                             \
    _Pragma("unroll") for (int jt = 0; jt < BT; ++jt) {                                              \
      _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                                \
        const vec<T, 4> w = *reinterpret_cast<const vec4_mem<T>*>(w_tile_ + c * LDX + 32 * jt + 8 * q + 4 * g); \
        _Pragma("unroll") for (int e = 0; e < 4; ++e) dA[jt][4 * q + e] *= (float)w[e];              \
      }                                                                                              \
      frag<T> okt[2][NT];                                                                            \
      _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2)                                               \
        _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                            \
          okt[s2][nt] = ld_free<T, true>(ku_tile_, LDK, 32 * nt, HD, 32 * jt + 16 * s2, c, g);       \
      __builtin_amdgcn_sched_barrier(0);                                                             \
      _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2) {                                             \
        const frag<T> fdz = chain<T>(dA[jt], s2);                                                    \
        _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) mma(dqu[nt], okt[s2][nt], fdz);            \
      }                                                                                              \
    }                                                                                                \
  } while (0)

    __syncthreads();   // 0
    for (int I = Ilast; I >= I0; --I) {
      const bool active = I >= Iw;
      // reverse state as of block I; the tile-consuming query kernel only reads those behind a
      // pair of blocks (odd I), the recomputing one all of them
      if (active && I <= a.s.nblk - 2 && (a.ds_mat == nullptr || (I & 1)))
        store_snap_tile<T, HD, NT>(gsnap + (gsnap_off(I) + kw0) * HD, G, c, g);
      __syncthreads();   // 1
      if (I < Ilast && I + 1 >= Iw) CASTLE_BK2_DQU(I + 1);   // finish the previous block
      // dA^T of this block, second term first: G (before this block) times Vu^T
#pragma unroll
      for (int jt = 0; jt < BT; ++jt) {
        zero(dA[jt]);
        if (active) {
          frag<T> ovu[KS];
#pragma unroll
          for (int s = 0; s < KS; ++s) ovu[s] = ld_chain<T>(s_vu, LDU, 32 * jt + c, 16 * s, g);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int s = 0; s < KS; ++s) mma(dA[jt], ovu[s], chain<T>(G[s / 2], s % 2));
        }
      }
#pragma unroll
      for (int it = 0; it < BT; ++it) {
        __syncthreads();   // 2, 3: sub-tile `it` is there
        const int i0 = I * kNB + 32 * it;
        if (active && i0 + 31 >= kw0) {
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            const int ic = 32 * it + 16 * s2;
            frag<T> odt[NT], oqt[NT], ott[BT];
            const frag<T> fp = ld_nat<T>(x_p, LDX, c, ic + 8 * g);
            const frag<T> fds = ld_nat<T>(x_ds, LDX, c, ic + 8 * g);
            const frag<T> fdsu = ld_nat<T>(x_dsu, LDX, c, ic + 8 * g);
            if (a.ds_mat != nullptr) {   // hand the tile to the query-stationary kernel: 1 KB contiguous per store
              const int64_t tile = ((int64_t)(kw0 / 32) * (a.s.Lp / 32) + i0 / 32) * 1024 + s2 * 512 + c * 16 + g * 8;
              __builtin_nontemporal_store(fds, reinterpret_cast<frag_mem<T>*>(ds_mat + tile));
              __builtin_nontemporal_store(fdsu, reinterpret_cast<frag_mem<T>*>(dsu_mat + tile));
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
              odt[nt] = ld_free<T, false>(s_do, LDK, 32 * nt, HD, ic, c, g);
              oqt[nt] = ld_free<T, false>(s_qc, LDK, 32 * nt, HD, ic, c, g);
            }
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
              if (jt <= it) ott[jt] = ld_free<T, false>(s_t, LDT, 32 * jt, kNB, ic, c, g);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
              mma(dvc[nt], odt[nt], fp);
              mma(dkc[nt], oqt[nt], fds);
              mma(G[nt], oqt[nt], fdsu);
            }
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
              if (jt <= it) mma(dA[jt], ott[jt], fdsu);
          }
        }
      }
      __syncthreads();   // 4
    }
    if (I0 >= Iw) CASTLE_BK2_DQU(I0);
#undef CASTLE_BK2_DQU
    if (k < L) {
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dkc, b, h) + (int64_t)k * a.dkc.sl, dkc, kLn2 * gun, g, a.s.rotary ? k : -1);
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dvc, b, h) + (int64_t)k * a.dvc.sl, dvc, gun, g);
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dqu, b, h) + (int64_t)k * a.dqu.sl, dqu, c0 * kLn2 * gun, g, a.s.rotary ? k : -1);
    }
  }
#undef CASTLE_BK2_STAGE_DECL
#undef CASTLE_BK2_STAGE_LOAD
#undef CASTLE_BK2_STAGE_STORE
#undef CASTLE_BK2_KU
#undef CASTLE_BK2_W
}

// ---------------------------------------------------------------------------
// Key-stationary backward for head dimensions above 64 (16-bit compute types) with two wave roles,
// in two launches: no wave can hold the four accumulator sets of its keys at d = 128, and a wave
// of either role must stay within half a SIMD's registers so that two of them share it.
//   launch 1 (bwd_keyw1_kernel):  score waves   Kc, Vc, -c1 Qu and the lookahead state of their 32 keys
//                                               in registers; per 32-query sub-tile the scores, P, dS,
//                                               dSu -> LDS for the partner and the dS / dSu tiles -> HBM
//                                 gradient waves  all staging of the block tiles; dVc, dKc
//   launch 2 (bwd_keyw2_kernel):  gate waves    staging; gate A of a block, then dZ = dA A (1 - A) and
//                                               dQu one block later
//                                 state waves   dSu fragments straight from the tiles; reverse state G
//                                               (snapshots), dA = G Vu^T + dSu^T T' -> LDS for the partner
// Pair (w, w + 4) owns keys kb*128 + 32 w .. + 31, as in bwd_key2_kernel.
template <typename T, int HD> constexpr int bwd_keyw1_lds_bytes() {
  int b = 3 * a16((int)sizeof(T) * kNB * lds_ld_tr<T>(HD));    // qc, do, ku
  b += a16((int)sizeof(T) * kNB * lds_ld_chain<T>(kNB));    // T'
  b += 2 * a16(4 * kNB);                                    // lse, delta
  b += 4 * 3 * a16((int)sizeof(T) * 32 * lds_ld<T>(kNB));   // P, dS, dSu per wave pair
  return b;
}
template <typename T, int HD> constexpr int bwd_keyw2_lds_bytes() {
  int b = 3 * a16((int)sizeof(T) * kNB * lds_ld_tr<T>(HD));    // qc, ku (two blocks)
  b += a16((int)sizeof(T) * kNB * lds_ld_chain<T>(HD));     // vu
  b += a16((int)sizeof(T) * kNB * lds_ld_chain<T>(kNB));    // T'
  b += 2 * 4 * a16((int)sizeof(T) * 32 * lds_ld<T>(kNB));   // dA per wave pair, two blocks
  return b;
}

template <typename T, typename TI, int HD>
__global__ __launch_bounds__(2 * kThreads, 1) void bwd_keyw1_kernel(BwdArgs a) {
  static_assert(sizeof(T) == 2 && HD > 64, "two-role kernel for wide heads: 16-bit operands");
  constexpr int KS = HD / 16;
  constexpr int NT = HD / 32;
  constexpr int BT = kNB / 32;
  constexpr int LDK = lds_ld_tr<T>(HD), LDT = lds_ld_chain<T>(kNB), LDX = lds_ld<T>(kNB);

  Carver cv{castle_smem};
  T* s_qc = cv.take<T>(kNB * LDK);
  T* s_do = cv.take<T>(kNB * LDK);
  T* s_ku = cv.take<T>(kNB * LDK);   // one buffer: only the gate reads it, between barriers 3 and 4
  T* s_t = cv.take<T>(kNB * LDT);
  float* s_lse = cv.take<float>(kNB);
  float* s_delta = cv.take<float>(kNB);
  T* s_x = cv.take<T>(4 * 3 * 32 * LDX);

  int kb, bh;
  work_item(a.s.B * a.s.H, kb, bh);
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const bool scorer = wave < 4;
  const int pw = wave & 3;
  const int L = a.s.L;
  const float c1 = a.s.scale * kLog2e;
  const float su_mul = a.ws.hdr->su_mul, gun = a.bhdr->grad_unscale;
  const int kw0 = kb * 128 + 32 * pw;
  const int k = kw0 + c;
  const int Iw = kw0 / kNB;
  const int I0 = (kb * 128) / kNB;
  const int Ilast = a.s.nblk - 1;
  T* x_p = s_x + pw * 3 * 32 * LDX;   // [key][query of the block]
  T* x_ds = x_p + 32 * LDX;
  T* x_dsu = x_ds + 32 * LDX;

  if (scorer) {
    const T* kc = prep_ptr<T>(a.ws.kc_p, bh, a.s.Lp, HD);
    const T* vc = prep_ptr<T>(a.ws.vc_p, bh, a.s.Lp, HD);
    const T* qu = prep_ptr<T>(a.ws.qu_p, bh, a.s.Lp, HD);
    const T* usnap = reinterpret_cast<const T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
    T* ds_mat = reinterpret_cast<T*>(a.ds_mat) + (int64_t)bh * a.s.Lp * a.s.Lp;
    T* dsu_mat = reinterpret_cast<T*>(a.dsu_mat) + (int64_t)bh * a.s.Lp * a.s.Lp;

    frag<T> fkc[KS], fvc[KS], fqu[KS], fub[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      fkc[s] = ldg_nat<T>(kc, HD, k, 16 * s + 8 * g, true);
      fvc[s] = ldg_nat<T>(vc, HD, k, 16 * s + 8 * g, true);
      fqu[s] = ldg_nat_scaled<T, T>(qu, HD, k, 16 * s + 8 * g, true, -c1);
      fub[s] = zero_frag<T>();
    }
    frag<T> fa[BT][2];
    // gate tiles A^T[j rows, k lanes] of source block J as operand fragments of its score tiles
#define CASTLE_BKW_GATE(J_)                                                                          \
  do {                                                                                               \
    _Pragma("unroll") for (int jt = 0; jt < BT; ++jt) {                                              \
      acc_t aT;                                                                                      \
      zero(aT);                                                                                      \
      _Pragma("unroll") for (int s0 = 0; s0 < KS; s0 += 4) {                                         \
        frag<T> oku[4];                                                                              \
        _Pragma("unroll") for (int u = 0; u < 4; ++u)                                                \
          oku[u] = ld_nat<T>(s_ku, LDK, 32 * jt + c, 16 * (s0 + u) + 8 * g);                         \
        __builtin_amdgcn_sched_barrier(0);                                                           \
        _Pragma("unroll") for (int u = 0; u < 4; ++u) mma(aT, oku[u], fqu[s0 + u]);                  \
      }                                                                                              \
      const int j0 = (J_) * kNB + 32 * jt;                                                           \
      _Pragma("unroll") for (int r = 0; r < 16; ++r) aT[r] = fast_rcp(1.f + fast_exp2(aT[r]));       \
      if (j0 <= kw0 + 31) { /* tile touches the diagonal: keep j > k only */                         \
        _Pragma("unroll") for (int r = 0; r < 16; ++r)                                               \
          if (j0 + acc_row(r, g) <= k) aT[r] = 0.f;                                                  \
      }                                                                                              \
      fa[jt][0] = chain<T>(aT, 0);                                                                   \
      fa[jt][1] = chain<T>(aT, 1);                                                                   \
    }                                                                                                \
  } while (0)

    if (Ilast > Iw) {
#pragma unroll
      for (int s = 0; s < KS; ++s) fub[s] = ldg_snap_nat<T>(usnap + (usnap_off(Ilast) + kw0) * HD, c, 16 * s + 8 * g);
    }
    __syncthreads();   // 0: first Ku tile staged
    if (Ilast >= Iw) CASTLE_BKW_GATE(Ilast);
    for (int I = Ilast; I >= I0; --I) {
      const bool active = I >= Iw;
      const bool inter = I > Iw;   // lookahead state from earlier blocks exists
      __syncthreads();   // 1: tiles staged
#pragma unroll
      for (int it = 0; it < BT; ++it) {
        const int i0 = I * kNB + 32 * it;
        if (active && i0 + 31 >= kw0) {   // else every query precedes every key of this wave
          acc_t sc, su, dp;   // sc starts from -lse, dp from -delta of its row
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const vec<float, 4> nl = *reinterpret_cast<const vec<float, 4>*>(s_lse + 32 * it + 8 * q + 4 * g);
            const vec<float, 4> nd = *reinterpret_cast<const vec<float, 4>*>(s_delta + 32 * it + 8 * q + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              sc[4 * q + e] = nl[e];
              dp[4 * q + e] = nd[e];
              su[4 * q + e] = 0.f;
            }
          }
#pragma unroll
          for (int s0 = 0; s0 < KS; s0 += 4) {   // operand fragments in batches of four
            frag<T> oq[4], od[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              oq[u] = ld_nat<T>(s_qc, LDK, 32 * it + c, 16 * (s0 + u) + 8 * g);
              od[u] = ld_nat<T>(s_do, LDK, 32 * it + c, 16 * (s0 + u) + 8 * g);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              mma(sc, oq[u], fkc[s0 + u]);
              mma(dp, od[u], fvc[s0 + u]);
              if (inter) mma(su, oq[u], fub[s0 + u]);
            }
          }
          {
            frag<T> ot[BT][2];
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
#pragma unroll
              for (int s2 = 0; s2 < 2; ++s2)
                if (jt <= it) ot[jt][s2] = ld_chain<T>(s_t, LDT, 32 * it + c, 32 * jt + 16 * s2, g);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
#pragma unroll
              for (int s2 = 0; s2 < 2; ++s2)
                if (jt <= it) mma(su, ot[jt][s2], fa[jt][s2]);
          }
          acc_t ds, dsu;
          if (i0 < kw0 + 31) {   // tile touches the diagonal: queries before the key see nothing
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if (i0 + acc_row(r, g) < k) sc[r] = -INFINITY;
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float sut = su[r] * su_mul;                 // log2(e) * Su
            const float sg = fast_rcp(1.f + fast_exp2(-sut));
            const float p = fast_exp2(__builtin_fmaf(-sut, sg, sc[r]));   // sc carries -lse
            const float dsv = p * dp[r];                      // dp carries -delta
            const float y = sut * kLn2;                       // true Su
            const float t = __builtin_fmaf(-y, sg, y);        // y (1 - sigmoid)
            const float sp = __builtin_fmaf(sg, t, sg);       // silu'(y)
            sc[r] = p;
            ds[r] = dsv;
            dsu[r] = -dsv * sp * su_mul;                      // gradient of the product built from vu * vu_scale
          }
          // For the partner through LDS; for the query-stationary kernel and the second launch as 32 x 32
          // tiles in HBM.  A tile is two runs of 16 queries, 16 bytes per key and lane half in each; the 8
          // values of a lane are its accumulator registers as they are (chained order: queries 4g..4g+3
          // and 8+4g..8+4g+3 of the run), so that one store instruction covers 1 KB of whole lines.
          const int64_t tile = ((int64_t)(kw0 / 32) * (a.s.Lp / 32) + i0 / 32) * 1024 + c * 16 + 8 * g;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int o = c * LDX + 32 * it + 8 * q + 4 * g;
            st4<T>(x_p + o, pack4<T>(sc, q));
            st4<T>(x_ds + o, pack4<T>(ds, q));
            st4<T>(x_dsu + o, pack4<T>(dsu, q));
          }
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            __builtin_nontemporal_store(chain<T>(ds, s2), reinterpret_cast<frag_mem<T>*>(ds_mat + tile + s2 * 512));
            __builtin_nontemporal_store(chain<T>(dsu, s2), reinterpret_cast<frag_mem<T>*>(dsu_mat + tile + s2 * 512));
          }
        }
        __syncthreads();   // 2, 3: sub-tile handed over
      }
      if (I > I0) {
        if (I - 1 > Iw) {   // lookahead state as of the next block: in flight behind the gate
#pragma unroll
          for (int s = 0; s < KS; ++s) fub[s] = ldg_snap_nat<T>(usnap + (usnap_off(I - 1) + kw0) * HD, c, 16 * s + 8 * g);
        }
        if (I - 1 >= Iw) CASTLE_BKW_GATE(I - 1);   // its Ku tile was staged before barrier 3
      }
      __syncthreads();   // 4: tiles free
    }
#undef CASTLE_BKW_GATE
  } else {
    const T* qc = prep_ptr<T>(a.ws.qc_p, bh, a.s.Lp, HD);
    const T* ku = prep_ptr<T>(a.ws.ku_p, bh, a.s.Lp, HD);
    const T* dout = prep_ptr<T>(a.dout_p, bh, a.s.Lp, HD);
    const T* tb = reinterpret_cast<const T*>(a.ws.t_blk) + (int64_t)bh * a.s.Lp * kNB;
    const float* lse = a.ws.lse + (int64_t)bh * a.s.Lp;
    const float* delta = a.delta + (int64_t)bh * a.s.Lp;
    const int tid = threadIdx.x - kThreads;   // thread index inside the role
    acc_t dvc[NT], dkc[NT];   // [n rows, k lanes]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) { zero(dvc[nt]); zero(dkc[nt]); }
    // These waves issue no global stores inside the loop, so the pieces of the next block can stay in
    // flight for a whole block without anything queueing behind them in the in-order memory counter.
    RowStage<T, T, kNB, HD> pku, pqc, pdo;
    RowStage<T, T, kNB, kNB> ptb;
    float plse = 0.f, pdelta = 0.f;
#define CASTLE_BKW_LOAD(I_)                                  \
  do {                                                       \
    const int64_t r_ = (int64_t)(I_) * kNB;                  \
    pku.load_flat(ku + r_ * HD, tid);                        \
    pqc.load_flat(qc + r_ * HD, tid);                        \
    pdo.load_flat(dout + r_ * HD, tid);                      \
    ptb.load_flat(tb + r_ * kNB, tid);                       \
    if (tid < kNB) {                                         \
      const int64_t i_ = r_ + tid;                           \
      plse = i_ < L ? lse[i_] : INFINITY;                    \
      pdelta = i_ < L ? delta[i_] : 0.f;                     \
    }                                                        \
  } while (0)
    CASTLE_BKW_LOAD(Ilast);
    pku.store(s_ku, LDK, tid);
    __syncthreads();   // 0
    for (int I = Ilast; I >= I0; --I) {
      const bool active = I >= Iw;
      pqc.store(s_qc, LDK, tid);
      pdo.store(s_do, LDK, tid);
      ptb.store_halves(s_t, LDT, tid);
      if (tid < kNB) {
        s_lse[tid] = -plse * kLog2e;
        s_delta[tid] = -pdelta;
      }
      __syncthreads();   // 1: tiles staged
      if (I > I0) CASTLE_BKW_LOAD(I - 1);   // in flight for the whole block
#pragma unroll
      for (int it = 0; it < BT; ++it) {
        if (it == 1 && I > I0) pku.store(s_ku, LDK, tid);   // the gate of block I finished before barrier 4 of block I + 1
        __syncthreads();   // 2, 3: sub-tile `it` is there
        const int i0 = I * kNB + 32 * it;
        if (active && i0 + 31 >= kw0) {
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            const int ic = 32 * it + 16 * s2;
            frag<T> odt[NT], oqt[NT];
            const frag<T> fp = ld_nat<T>(x_p, LDX, c, ic + 8 * g);
            const frag<T> fds = ld_nat<T>(x_ds, LDX, c, ic + 8 * g);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
              odt[nt] = ld_free<T, false>(s_do, LDK, 32 * nt, HD, ic, c, g);
              oqt[nt] = ld_free<T, false>(s_qc, LDK, 32 * nt, HD, ic, c, g);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
              mma(dvc[nt], odt[nt], fp);
              mma(dkc[nt], oqt[nt], fds);
            }
          }
        }
      }
      __syncthreads();   // 4
    }
#undef CASTLE_BKW_LOAD
    if (k < L) {
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dkc, b, h) + (int64_t)k * a.dkc.sl, dkc, kLn2 * gun, g, a.s.rotary ? k : -1);
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dvc, b, h) + (int64_t)k * a.dvc.sl, dvc, gun, g);
    }
  }
}

template <typename T, typename TI, int HD>
__global__ __launch_bounds__(2 * kThreads, 1) void bwd_keyw2_kernel(BwdArgs a) {
  static_assert(sizeof(T) == 2 && HD > 64, "two-role kernel for wide heads: 16-bit operands");
  constexpr int KS = HD / 16;
  constexpr int NT = HD / 32;
  constexpr int BT = kNB / 32;
  constexpr int LDK = lds_ld_tr<T>(HD), LDU = lds_ld_chain<T>(HD), LDT = lds_ld_chain<T>(kNB), LDX = lds_ld<T>(kNB);
  // dA crosses the LDS as a 16-bit value: a quarter of it, so that it needs no more range than
  // dZ = dA A (1 - A) <= dA / 4, which is a 16-bit MFMA operand in every variant of this kernel
  constexpr float kHand = 0.25f, kUnhand = 4.f;

  Carver cv{castle_smem};
  T* s_qc = cv.take<T>(kNB * LDK);
  T* s_ku0 = cv.take<T>(kNB * LDK);
  T* s_ku1 = cv.take<T>(kNB * LDK);
  T* s_vu = cv.take<T>(kNB * LDU);
  T* s_t = cv.take<T>(kNB * LDT);
  T* s_da = cv.take<T>(2 * 4 * 32 * LDX);

  int kb, bh;
  work_item(a.s.B * a.s.H, kb, bh);
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const bool gater = wave < 4;
  const int pw = wave & 3;
  const int L = a.s.L;
  const float c0 = a.s.scale, c1 = a.s.scale * kLog2e;
  const float gun = a.bhdr->grad_unscale;
  const int kw0 = kb * 128 + 32 * pw;
  const int k = kw0 + c;
  const int Iw = kw0 / kNB;
  const int I0 = (kb * 128) / kNB;
  const int Ilast = a.s.nblk - 1;
  T* x_da = s_da + pw * 32 * LDX;   // [key][source of the block], + 4*32*LDX for odd blocks
#define CASTLE_BKW_KU(I_) (((I_) & 1) ? s_ku1 : s_ku0)
#define CASTLE_BKW_DA(I_) (x_da + ((I_) & 1) * 4 * 32 * LDX)

  if (gater) {
    const T* qc = prep_ptr<T>(a.ws.qc_p, bh, a.s.Lp, HD);
    const T* qu = prep_ptr<T>(a.ws.qu_p, bh, a.s.Lp, HD);
    const T* ku = prep_ptr<T>(a.ws.ku_p, bh, a.s.Lp, HD);
    const T* vu = prep_ptr<T>(a.ws.vu_p, bh, a.s.Lp, HD);
    const T* tb = reinterpret_cast<const T*>(a.ws.t_blk) + (int64_t)bh * a.s.Lp * kNB;
    frag<T> fqu[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) fqu[s] = ldg_nat_scaled<T, T>(qu, HD, k, 16 * s + 8 * g, true, -c1);
    acc_t dqu[NT];   // [n rows, k lanes]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero(dqu[nt]);
    vec<T, 4> w[BT][4];   // 4 A (1 - A) of the block whose dA is still to come, [j rows, k lanes], packed
#pragma unroll
    for (int jt = 0; jt < BT; ++jt)
#pragma unroll
      for (int q = 0; q < 4; ++q) w[jt][q] = vec<T, 4>{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
    RowStage<T, T, kNB, HD> pku, pqc, pvu;
    RowStage<T, T, kNB, kNB> ptb;
    // The pieces of the next block are requested in four portions spread over the block: the CU takes
    // one 1 KB wave load per 16 cycles, and a burst of all 56 of them held every wave of the workgroup
    // up for more than a thousand cycles behind barrier 1.
#define CASTLE_BKW_LOAD(I_, PORTION)                                        \
  do {                                                                      \
    const int64_t r_ = (int64_t)(I_) * kNB;                                 \
    if ((PORTION) == 0 || (PORTION) < 0) pku.load_flat(ku + r_ * HD);       \
    if ((PORTION) == 1 || (PORTION) < 0) pqc.load_flat(qc + r_ * HD);       \
    if ((PORTION) == 2 || (PORTION) < 0) pvu.load_flat(vu + r_ * HD);       \
    if ((PORTION) == 3 || (PORTION) < 0) ptb.load_flat(tb + r_ * kNB);      \
  } while (0)
    // dZ^T = dA^T * A (1 - A)  ->  dQu, for source block J: its Ku tile is still in its buffer
#define CASTLE_BKW_DQU(J_, JT_)                                                                      \
  do {                                                                                               \
    const T* ku_tile_ = CASTLE_BKW_KU(J_);                                                           \
    const T* da_tile_ = CASTLE_BKW_DA(J_);                                                           \
    constexpr int jt = (JT_);                                                                        \
    acc_t dz;                                                                                        \
    _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                                  \
      const vec<T, 4> d4 = *reinterpret_cast<const vec4_mem<T>*>(da_tile_ + c * LDX + 32 * jt + 8 * q + 4 * g); \
      _Pragma("unroll") for (int e = 0; e < 4; ++e) dz[4 * q + e] = (float)d4[e] * (float)w[jt][q][e]; \
    }                                                                                                \
    _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2) {                                               \
      frag<T> okt[NT];                                                                               \
      _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                              \
        okt[nt] = ld_free<T, true>(ku_tile_, LDK, 32 * nt, HD, 32 * jt + 16 * s2, c, g);             \
      __builtin_amdgcn_sched_barrier(0);                                                             \
      const frag<T> fdz = chain<T>(dz, s2);                                                          \
      _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) mma(dqu[nt], okt[nt], fdz);                  \
    }                                                                                                \
  } while (0)

    static_assert(BT == 2, "the portions below are placed around two gate tiles");
    CASTLE_BKW_LOAD(Ilast, -1);
    for (int I = Ilast; I >= I0; --I) {
      // every wave has passed the end barrier of block I + 1: its tiles are free, and so is the Ku
      // buffer of block I + 2, which block I takes over
      pqc.store(s_qc, LDK);
      pvu.store_halves(s_vu, LDU);
      ptb.store_halves(s_t, LDT);
      pku.store(CASTLE_BKW_KU(I), LDK);
      __syncthreads();   // 1: tiles staged
      const bool more = I > I0, owed = I < Ilast && I + 1 >= Iw;
      if (more) CASTLE_BKW_LOAD(I - 1, 0);
      if (owed) CASTLE_BKW_DQU(I + 1, 0);   // finish the previous block
      if (more) CASTLE_BKW_LOAD(I - 1, 1);
      if (owed) CASTLE_BKW_DQU(I + 1, 1);
      if (more) CASTLE_BKW_LOAD(I - 1, 2);
      if (I >= Iw) {   // gate of this block: 4 A (1 - A) stays in registers until its dA arrives
        const T* ku_tile = CASTLE_BKW_KU(I);
#pragma unroll
        for (int jt = 0; jt < BT; ++jt) {
          if (jt == 1 && more) CASTLE_BKW_LOAD(I - 1, 3);
          acc_t aT;
          zero(aT);
#pragma unroll
          for (int s0 = 0; s0 < KS; s0 += 2) {   // operand fragments in pairs: this role is at the register limit
            frag<T> oku[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) oku[u] = ld_nat<T>(ku_tile, LDK, 32 * jt + c, 16 * (s0 + u) + 8 * g);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < 2; ++u) mma(aT, oku[u], fqu[s0 + u]);
          }
          const int j0 = I * kNB + 32 * jt;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float av = fast_rcp(1.f + fast_exp2(aT[r]));
            aT[r] = kUnhand * __builtin_fmaf(-av, av, av);
          }
          if (j0 <= kw0 + 31) {   // tile touches the diagonal: keep j > k only
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if (j0 + acc_row(r, g) <= k) aT[r] = 0.f;
          }
#pragma unroll
          for (int q = 0; q < 4; ++q) w[jt][q] = pack4<T>(aT, q);
        }
      }
      __syncthreads();   // 2: block done, dA of block I written
    }
    if (I0 >= Iw) {
      CASTLE_BKW_DQU(I0, 0);
      CASTLE_BKW_DQU(I0, 1);
    }
#undef CASTLE_BKW_LOAD
#undef CASTLE_BKW_DQU
    if (k < L) store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dqu, b, h) + (int64_t)k * a.dqu.sl, dqu, c0 * kLn2 * gun, g, a.s.rotary ? k : -1);
  } else {
    T* gsnap = reinterpret_cast<T*>(a.gsnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
    const T* dsu_tiles = reinterpret_cast<const T*>(a.dsu_mat) + (int64_t)bh * a.s.Lp * a.s.Lp +
                         (int64_t)(kw0 / 32) * (a.s.Lp / 32) * 1024 + c * 16 + 8 * g;
    acc_t G[NT];   // [n rows, k lanes]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero(G[nt]);
    // dSu fragments of a block's sub-tiles straight from the tiles (lane = key, 8 queries in the
    // chained order the first launch stored them in); those of the next block are requested a block ahead
    frag<T> tdsu[BT][2], tnext[BT][2];
#define CASTLE_BKW_TILES(DST, I_)                                                                     \
  do {                                                                                                \
    _Pragma("unroll") for (int it = 0; it < BT; ++it) {                                               \
      const int i0_ = (I_) * kNB + 32 * it;                                                           \
      _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2)                                                \
        DST[it][s2] = ((I_) >= Iw && i0_ + 31 >= kw0)                                                 \
                          ? __builtin_nontemporal_load(reinterpret_cast<const frag_mem<T>*>(dsu_tiles + (int64_t)(i0_ / 32) * 1024 + s2 * 512)) \
                          : zero_frag<T>();                                                           \
    }                                                                                                 \
  } while (0)
    CASTLE_BKW_TILES(tnext, Ilast);
    for (int I = Ilast; I >= I0; --I) {
      const bool active = I >= Iw;
      // the fragments requested a block ago are waited for here, ahead of the stores below: behind
      // them the wait would cover the stores too
#pragma unroll
      for (int it = 0; it < BT; ++it)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          tdsu[it][s2] = tnext[it][s2];
          asm volatile("" : "+v"(tdsu[it][s2]));
        }
      // reverse state as of block I; the query-stationary kernel reads those behind a pair of blocks
      if (active && I <= a.s.nblk - 2 && (I & 1)) store_snap_tile<T, HD, NT>(gsnap + (gsnap_off(I) + kw0) * HD, G, c, g);
      __syncthreads();   // 1: tiles staged
      if (!active && I > I0) CASTLE_BKW_TILES(tnext, I - 1);
      if (active) {
        // dA^T[j rows, k lanes] of this block, second term first: G (before this block) times Vu^T
        acc_t dA[BT];
#pragma unroll
        for (int jt = 0; jt < BT; ++jt) {
          zero(dA[jt]);
#pragma unroll
          for (int s0 = 0; s0 < KS; s0 += 4) {
            frag<T> ovu[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) ovu[u] = ld_chain<T>(s_vu, LDU, 32 * jt + c, 16 * (s0 + u), g);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < 4; ++u) mma(dA[jt], ovu[u], chain<T>(G[(s0 + u) / 2], (s0 + u) % 2));
          }
        }
        if (I > I0) CASTLE_BKW_TILES(tnext, I - 1);   // behind the partner's requests, which come right after barrier 1
#pragma unroll
        for (int it = 0; it < BT; ++it) {
          const int i0 = I * kNB + 32 * it;
          if (i0 + 31 < kw0) continue;   // every query precedes every key of this wave
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            const int ic = 32 * it + 16 * s2;
            frag<T> oqt[NT], ott[BT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) oqt[nt] = ld_free<T, true>(s_qc, LDK, 32 * nt, HD, ic, c, g);
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
              if (jt <= it) ott[jt] = ld_free<T, true>(s_t, LDT, 32 * jt, kNB, ic, c, g);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) mma(G[nt], oqt[nt], tdsu[it][s2]);
#pragma unroll
            for (int jt = 0; jt < BT; ++jt)
              if (jt <= it) mma(dA[jt], ott[jt], tdsu[it][s2]);
          }
        }
        T* da_tile = CASTLE_BKW_DA(I);
#pragma unroll
        for (int jt = 0; jt < BT; ++jt) {
#pragma unroll
          for (int r = 0; r < 16; ++r) dA[jt][r] *= kHand;
#pragma unroll
          for (int q = 0; q < 4; ++q) st4<T>(da_tile + c * LDX + 32 * jt + 8 * q + 4 * g, pack4<T>(dA[jt], q));
        }
      }
      __syncthreads();   // 2: block done
    }
#undef CASTLE_BKW_TILES
  }
#undef CASTLE_BKW_KU
#undef CASTLE_BKW_DA
}

// ---------------------------------------------------------------------------
constexpr int kCK = 32;   // keys per chunk in the query-stationary backward

template <typename T, int HD> constexpr int bwd_query_lds_bytes() {
  int b = 7 * a16((int)sizeof(T) * kCK * lds_ld<T>(HD));           // kc, vc, qu, ub[2], g[2]
  b += 2 * a16((int)sizeof(T) * 128 * lds_ld_chain<T>(kCK));       // A^T [j][k], dSu^T [i][k]
  // epilogue (reuses the same memory): vu[2], qc[2], dT [i][j] for both blocks
  int e = 4 * a16((int)sizeof(T) * kNB * lds_ld<T>(HD)) + 2 * a16((int)sizeof(T) * kNB * lds_ld_chain<T>(kNB));
  return b > e ? b : e;
}

// PART: 0 = all outputs (d <= 64); 1 = dQc; 2 = dKu, dVu (see bwd_key_kernel).
template <typename T, typename TI, int HD, int PART>
__global__ __launch_bounds__(kThreads, 1) void bwd_query_kernel(BwdArgs a) {
  constexpr bool DO_Q = PART != 2, DO_S = PART != 1;
  constexpr int KS = HD / 16;
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr int NT = HDP / 32;
  constexpr int BT = kNB / 32;
  constexpr int TS = kNB / 16;   // 16-deep steps across a block
  constexpr int CKT = kCK / 32;  // 32-key sub-tiles per chunk
  constexpr int QB = 128;
  constexpr int NQ = QB / kNB;
  constexpr int LDK = lds_ld<T>(HD), LDC = lds_ld_chain<T>(kCK), LDT = lds_ld_chain<T>(kNB);

  Carver cv{castle_smem};
  T* s_kc = cv.take<T>(kCK * LDK);
  T* s_vc = cv.take<T>(kCK * LDK);
  T* s_qu = cv.take<T>(kCK * LDK);
  T* s_ub0 = cv.take<T>(kCK * LDK);
  T* s_ub1 = cv.take<T>(kCK * LDK);
  T* s_g0 = cv.take<T>(kCK * LDK);
  T* s_g1 = cv.take<T>(kCK * LDK);
  T* s_at = cv.take<T>(QB * LDC);     // gate, [source j][key k]
  T* s_dsut = cv.take<T>(QB * LDC);   // dSu,  [query i][key k]

  int rank, bh;
  work_item(a.s.B * a.s.H, rank, bh);
  const int qb = a.s.Lp / 128 - 1 - rank;   // the last row block meets the most keys
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const int L = a.s.L;
  const float c0 = a.s.scale, c1 = a.s.scale * kLog2e;
  const float su_mul = a.ws.hdr->su_mul, gun = a.bhdr->grad_unscale, vu_scale = a.ws.hdr->vu_scale;
  const int i0w = qb * QB + 32 * wave;
  const int i = i0w + c;                      // this lane's row: a query in phase 1, a source in phase 2
  const int Ifirst = (qb * QB) / kNB;
  const int Iw = i0w / kNB;
  const int qw = Iw - Ifirst;                 // which of the workgroup's blocks
  const int jw = 32 * wave;                   // rows of this wave inside the 128-row exchange tiles
  const int cb = (jw / kNB) * kNB;            // first row of its block there
  const int lw = jw % kNB;                    // offset of the wave inside its block
  const int nintra = (lw + 32) / 16;          // steps covering sources j <= i
  const int ifirst = lw / 16;                 // first step covering queries i >= j
  const bool has_g = Iw <= a.s.nblk - 2;
  const T* s_ubw = qw == 0 ? s_ub0 : s_ub1;
  const T* s_gw = qw == 0 ? s_g0 : s_g1;

  const T* qc = prep_ptr<T>(a.ws.qc_p, bh, a.s.Lp, HD);
  const T* kc = prep_ptr<T>(a.ws.kc_p, bh, a.s.Lp, HD);
  const T* vc = prep_ptr<T>(a.ws.vc_p, bh, a.s.Lp, HD);
  const T* qu = prep_ptr<T>(a.ws.qu_p, bh, a.s.Lp, HD);
  const T* ku = prep_ptr<T>(a.ws.ku_p, bh, a.s.Lp, HD);
  const T* vu = prep_ptr<T>(a.ws.vu_p, bh, a.s.Lp, HD);
  const T* dout = prep_ptr<T>(a.dout_p, bh, a.s.Lp, HD);
  const T* tb = reinterpret_cast<const T*>(a.ws.t_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* ttb = reinterpret_cast<const T*>(a.ws.tt_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* usnap = reinterpret_cast<const T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  const T* gsnap = reinterpret_cast<const T*>(a.gsnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;

  frag<T> fqc[KS], fdo[KS], fku[KS], fvu[KS], ft[TS], ftt[TS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    fqc[s] = ldg_nat<T>(qc, HD, i, 16 * s + 8 * g, true);
    fdo[s] = ldg_nat<T>(dout, HD, i, 16 * s + 8 * g, true);
    fku[s] = ldg_nat_scaled<T, T>(ku, HD, i, 16 * s + 8 * g, true, -c1);
    fvu[s] = ldg_nat<T>(vu, HD, i, 16 * s + 8 * g, true);
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

  // staging: every thread carries one 16-byte piece of each of the 7 tiles of the next chunk
  RowStage<T, T, kCK, HD> pkc, pvc, pqu;
  SnapStage<T, kCK, HD> pu0, pu1, pg0, pg1;
  const int blk0 = Ifirst, blk1 = Ifirst + 1;
#define CASTLE_BQ_LOAD(K0)                                                                                      \
  do {                                                                                                          \
    const int kb_ = (K0) / kNB;                                                                                 \
    pkc.load_flat(kc + (int64_t)(K0) * HD);                                                                             \
    pvc.load_flat(vc + (int64_t)(K0) * HD);                                                                             \
    pqu.load_flat(qu + (int64_t)(K0) * HD);                                                                             \
    if (kb_ < blk0) pu0.load(usnap + (usnap_off(blk0) + (K0)) * HD);                          \
    if (kb_ < blk1 && blk1 < a.s.nblk) pu1.load(usnap + (usnap_off(blk1) + (K0)) * HD);        \
    if (DO_S && kb_ <= blk0 && blk0 <= a.s.nblk - 2) pg0.load(gsnap + (gsnap_off(blk0) + (K0)) * HD);  \
    if (DO_S && kb_ <= blk1 && blk1 <= a.s.nblk - 2) pg1.load(gsnap + (gsnap_off(blk1) + (K0)) * HD);  \
  } while (0)

  int kend = qb * QB + QB;
  if (kend > a.s.Lp) kend = a.s.Lp;
  constexpr bool PF = HD <= 64;   // d = 128 has no registers to spare for a chunk in flight
  if (PF) CASTLE_BQ_LOAD(0);
  for (int k0 = 0; k0 < kend; k0 += kCK) {
    const int Kb = k0 / kNB;
    __syncthreads();
    if (!PF) CASTLE_BQ_LOAD(k0);
    pkc.store(s_kc, LDK);
    pvc.store(s_vc, LDK);
    pqu.store(s_qu, LDK);
    if (Kb < blk0) pu0.store(s_ub0, LDK);
    if (Kb < blk1 && blk1 < a.s.nblk) pu1.store(s_ub1, LDK);
    if (DO_S && Kb <= blk0 && blk0 <= a.s.nblk - 2) pg0.store(s_g0, LDK);
    if (DO_S && Kb <= blk1 && blk1 <= a.s.nblk - 2) pg1.store(s_g1, LDK);
    if (PF && k0 + kCK < kend) CASTLE_BQ_LOAD(k0 + kCK);   // in flight while this chunk is processed
    __syncthreads();
    const bool active = Kb <= Iw;

    // phase 0: gate tiles A[k rows, j lanes] for this wave's 32 source rows, shared as A^T[j][k]
    acc_t aK[CKT];
#pragma unroll
    for (int kt = 0; kt < CKT; ++kt) {
      zero(aK[kt]);
      if (!active) continue;
      {
        frag<T> oqu[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) oqu[s] = ld_nat<T>(s_qu, LDK, 32 * kt + c, 16 * s + 8 * g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS; ++s) mma(aK[kt], oqu[s], fku[s]);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) aK[kt][r] = fast_rcp(1.f + fast_exp2(aK[kt][r]));
      if (k0 + 32 * kt + 31 >= i0w) {   // sub-tile reaches the diagonal: keep j > k only
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (i <= k0 + 32 * kt + acc_row(r, g)) aK[kt][r] = 0.f;
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) st4<T>(s_at + (jw + c) * LDC + 32 * kt + 8 * q + 4 * g, pack4<T>(aK[kt], q));
    }
    __syncthreads();

    // phase 1: this lane's row is a query
#pragma unroll
    for (int kt = 0; kt < CKT; ++kt) {
      const int ks = k0 + 32 * kt;
      if (!(active && ks <= i0w + 31)) continue;
      acc_t sc, su, dp;
      zero(sc); zero(su); zero(dp);
      {
        // all operand fragments of this group are requested before the first MFMA
        frag<T> okc[KS], oub[KS], ovc[KS], oat[TS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          okc[s] = ld_nat<T>(s_kc, LDK, 32 * kt + c, 16 * s + 8 * g);
          ovc[s] = ld_nat<T>(s_vc, LDK, 32 * kt + c, 16 * s + 8 * g);
          oub[s] = ld_nat<T>(s_ubw, LDK, 32 * kt + c, 16 * s + 8 * g);
        }
#pragma unroll
        for (int s = 0; s < TS; ++s) oat[s] = ld_free<T, false>(s_at + cb * LDC, LDC, 32 * kt, kCK, 16 * s, c, g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          mma(sc, okc[s], fqc[s]);
          mma(dp, ovc[s], fdo[s]);
        }
        if (Kb < Iw) {
#pragma unroll
          for (int s = 0; s < KS; ++s) mma(su, oub[s], fqc[s]);
        }
#pragma unroll
        for (int s = 0; s < TS; ++s)
          if (s < nintra) mma(su, oat[s], ft[s]);
      }
      acc_t ds, dsu;
      const bool diag = ks + 31 > i0w;   // sub-tile reaches the diagonal
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float sut = su[r] * su_mul;                 // log2(e) * Su
        const float sg = fast_rcp(1.f + fast_exp2(-sut));
        const float x = __builtin_fmaf(-sut, sg, sc[r]);
        float p = fast_exp2(x - lse2);
        if (diag && ks + acc_row(r, g) > i) p = 0.f;
        const float dsv = p * (dp[r] - dlt);
        const float y = sut * kLn2;                       // true Su
        const float t = __builtin_fmaf(-y, sg, y);
        const float sp = __builtin_fmaf(sg, t, sg);
        ds[r] = dsv;
        dsu[r] = -dsv * sp * su_mul;                      // gradient of the product built from vu * vu_scale
      }
      if constexpr (DO_S) {
#pragma unroll
        for (int q = 0; q < 4; ++q) st4<T>(s_dsut + (jw + c) * LDC + 32 * kt + 8 * q + 4 * g, pack4<T>(dsu, q));
      }
      {
        frag<T> okt[2][NT], out[2][NT], oat[2][BT];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const int kc0 = 32 * kt + 16 * s2;
          if constexpr (DO_Q) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
              okt[s2][nt] = ld_free<T, true>(s_kc, LDK, 32 * nt, HD, kc0, c, g);
              out[s2][nt] = ld_free<T, true>(s_ubw, LDK, 32 * nt, HD, kc0, c, g);
            }
          }
#pragma unroll
          for (int jt = 0; jt < BT; ++jt) oat[s2][jt] = ld_chain<T>(s_at, LDC, cb + 32 * jt + c, kc0, g);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const frag<T> fds = chain<T>(ds, s2), fdsu = chain<T>(dsu, s2);
          if constexpr (DO_Q) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
              mma(dqc[nt], okt[s2][nt], fds);
              if (Kb < Iw) mma(dqc[nt], out[s2][nt], fdsu);
            }
          }
#pragma unroll
          for (int jt = 0; jt < BT; ++jt)
            if (32 * jt < lw + 32) mma(dtacc[jt], oat[s2][jt], fdsu);
        }
      }
    }
    __syncthreads();

    // phase 2: this lane's row is a lookahead source j; needs some key k < j
#pragma unroll
    for (int kt = 0; kt < (DO_S ? CKT : 0); ++kt) {
      const int ks = k0 + 32 * kt;
      if (!(active && ks < i0w + 31)) continue;
      acc_t dA;
      zero(dA);
      frag<T> oqt[2][NT], ogt[2][NT];
      {
        frag<T> ods[TS], og[KS];
#pragma unroll
        for (int s = 0; s < TS; ++s) ods[s] = ld_free<T, false>(s_dsut + cb * LDC, LDC, 32 * kt, kCK, 16 * s, c, g);
#pragma unroll
        for (int s = 0; s < KS; ++s) og[s] = has_g ? ld_nat<T>(s_gw, LDK, 32 * kt + c, 16 * s + 8 * g) : zero_frag<T>();
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            oqt[s2][nt] = ld_free<T, true>(s_qu, LDK, 32 * nt, HD, 32 * kt + 16 * s2, c, g);
            ogt[s2][nt] = has_g ? ld_free<T, true>(s_gw, LDK, 32 * nt, HD, 32 * kt + 16 * s2, c, g) : zero_frag<T>();
          }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < TS; ++s)
          if (s >= ifirst) mma(dA, ods[s], ftt[s]);
#pragma unroll
        for (int s = 0; s < KS; ++s) mma(dA, og[s], fvu[s]);   // og is zero where no reverse state exists
      }
      acc_t dz;
#pragma unroll
      for (int r = 0; r < 16; ++r) dz[r] = dA[r] * aK[kt][r] * (1.f - aK[kt][r]);
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const frag<T> fdz = chain<T>(dz, s2), fa = chain<T>(aK[kt], s2);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          mma(dku[nt], oqt[s2][nt], fdz);
          mma(dvu[nt], ogt[s2][nt], fa);
        }
      }
    }
  }
#undef CASTLE_BQ_LOAD

  // ---- epilogue: in-block terms dT = tril(dTacc):  dqc += dT Vu,  dvu += dT^T Qc' ------------
  __syncthreads();
  Carver ce{castle_smem};
  T* e_vu0 = ce.take<T>(kNB * LDK);
  T* e_vu1 = ce.take<T>(kNB * LDK);
  T* e_qc0 = ce.take<T>(kNB * LDK);
  T* e_qc1 = ce.take<T>(kNB * LDK);
  T* e_dt0 = ce.take<T>(kNB * LDT);   // dT, [query i][source j] (block local)
  T* e_dt1 = ce.take<T>(kNB * LDT);
  {
    RowStage<T, T, kNB, HD> st;
    st.load(vu, HD, (int64_t)blk0 * kNB, kNoRowLimit); st.store(e_vu0, LDK);
    st.load(vu, HD, (int64_t)blk1 * kNB, kNoRowLimit); st.store(e_vu1, LDK);
    st.load(qc, HD, (int64_t)blk0 * kNB, kNoRowLimit); st.store(e_qc0, LDK);
    st.load(qc, HD, (int64_t)blk1 * kNB, kNoRowLimit); st.store(e_qc1, LDK);
  }
  const T* e_vuw = qw == 0 ? e_vu0 : e_vu1;
  const T* e_qcw = qw == 0 ? e_qc0 : e_qc1;
  T* e_dtw = qw == 0 ? e_dt0 : e_dt1;
  // dT^T[j rows, i lanes] masked to j <= i, shared as dT[i][j] for the source-side product
#pragma unroll
  for (int jt = 0; jt < BT; ++jt) {
#pragma unroll
    for (int r = 0; r < 16; ++r)
      if (32 * jt + acc_row(r, g) > lw + c) dtacc[jt][r] = 0.f;
#pragma unroll
    for (int q = 0; q < 4; ++q) st4<T>(e_dtw + (lw + c) * LDT + 32 * jt + 8 * q + 4 * g, pack4<T>(dtacc[jt], q));
  }
  __syncthreads();
#pragma unroll
  for (int jt = 0; jt < (DO_Q ? BT : 0); ++jt) {
    if (32 * jt >= lw + 32) continue;
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const frag<T> fdt = chain<T>(dtacc[jt], s2);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        mma(dqc[nt], ld_free<T, true>(e_vuw, LDK, 32 * nt, HD, 32 * jt + 16 * s2, c, g), fdt);
    }
  }
#pragma unroll
  for (int s = 0; s < (DO_S ? TS : 0); ++s) {
    if (s < ifirst) continue;
    // B operand: source j = lw + c on lanes, queries i = 16 s .. natural order, from dT[i][j]
    const frag<T> fdt = ld_free<T, false>(e_dtw, LDT, lw, kNB, 16 * s, c, g);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      mma(dvu[nt], ld_free<T, false>(e_qcw, LDK, 32 * nt, HD, 16 * s, c, g), fdt);
  }
  if (i < L) {
    if constexpr (DO_Q) store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dqc, b, h) + (int64_t)i * a.dqc.sl, dqc, c0 * gun, g, a.s.rotary ? i : -1);
    if constexpr (DO_S) {
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dku, b, h) + (int64_t)i * a.dku.sl, dku, c0 * kLn2 * gun, g, a.s.rotary ? i : -1);
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dvu, b, h) + (int64_t)i * a.dvu.sl, dvu, kLn2 * gun * vu_scale, g, a.s.rotary ? i : -1);
    }
  }
}

// ---------------------------------------------------------------------------
// Query-stationary backward that consumes the dS / dSu tiles written by the key-stationary kernels
// (16-bit compute types): no score recomputation, only the gate.
//   row = query i:   dQc += dS Kc + dSu U_I,  dT^T += A^T dSu^T
//   row = source j:  dA = dSu^T T' + G' Vu^T,  dZ = dA A (1 - A),  dKu += dZ^T Qu,  dVu += A^T G'
template <typename T> constexpr int kLdD = 128 + 8;   // dS / dSu tiles [key][128 queries]
template <typename T> constexpr int kLdA = kCK + 8;   // gate tile [128 sources][key]
template <typename T> constexpr int kLdT2 = 128 + 4;  // dT of the row pair [128 queries][128 sources]
template <typename T> constexpr int kLdTT = 128 + 8;  // T'^T rows of the pair [128 sources][128 queries] (bwd_queryw_kernel)
template <typename T, int HD> constexpr int bwd_query2_lds_bytes() {
  int b = 4 * a16((int)sizeof(T) * kCK * lds_ld_tr<T>(HD));       // kc, qu, ub, g
  b += a16((int)sizeof(T) * 128 * kLdA<T>);                       // A^T [j][k]
  b += 2 * a16((int)sizeof(T) * kCK * kLdD<T>);                   // dS, dSu [k][i]
  int e = 2 * a16((int)sizeof(T) * 128 * lds_ld_tr<T>(HD)) + a16((int)sizeof(T) * 128 * kLdT2<T>);
  return b > e ? b : e;
}

// Staging of the 4 consecutive 32x32 tiles (8 KB) that one chunk of 32 keys shares with the 128
// queries of a workgroup, one 16-byte piece per thread (512 threads).  Every wave instruction
// reads 1 KB contiguous; within 16 lanes the LDS rows differ, which keeps the stores conflict free.
// CHAINED: the 8 values of a piece are queries 4g..4g+3 and 8+4g..8+4g+3 of their run of 16 (tiles
// written from accumulator registers by bwd_keyw1_kernel); the LDS tile is in natural order either way.
template <typename T, bool CHAINED>
struct TileStage {
  vec<T, 8> r;
  __device__ __forceinline__ void load(const T* src) {
    const int slab = threadIdx.x >> 6, l = threadIdx.x & 63;       // slab = 2 * tile + s2
    const int g = (l >> 4) & 1, k = (l & 15) + 16 * (l >> 5);
    r = __builtin_nontemporal_load(reinterpret_cast<const frag_mem<T>*>(src + slab * 512 + k * 16 + g * 8));   // read once
  }
  __device__ __forceinline__ void store(T* dst) const {
    const int slab = threadIdx.x >> 6, l = threadIdx.x & 63;
    const int g = (l >> 4) & 1, k = (l & 15) + 16 * (l >> 5);
    if constexpr (CHAINED) {
      vec<T, 4> lo, hi;
#pragma unroll
      for (int e = 0; e < 4; ++e) { lo[e] = r[e]; hi[e] = r[4 + e]; }
      st4<T>(dst + k * kLdD<T> + 16 * slab + 4 * g, lo);
      st4<T>(dst + k * kLdD<T> + 16 * slab + 8 + 4 * g, hi);
    } else {
      *reinterpret_cast<frag_mem<T>*>(dst + k * kLdD<T> + 16 * slab + 8 * g) = r;
    }
  }
};

// 512 threads, two wave roles over the same 128 rows = one PAIR of 64-row blocks (2 qb, 2 qb + 1);
// wave pair (w, w + 4) owns rows 32 w ..:
//   waves 0-3, row = lookahead source j:  gate A, dA, dZ, dKu
//   waves 4-7, row = query i: dQc, dT;  row = source j: dVu (gate read back from the shared tile)
// Keys are streamed in chunks of 32 (three barriers per chunk); two waves share a SIMD.
// The pair is handled as ONE block with respect to the two states: the lookahead state U is the
// one at the start of the pair and the reverse state G' the one behind the pair (one snapshot tile
// of each per chunk instead of two), and what the states of the inner block boundary would have
// carried goes through the pair's own 128 x 128 quarter-filled dT / T' instead:
//   dA[k,j]  = sum_{i in pair, i >= j} dSu[i,k] T'[i,j] + G'[k] . vu_j
//   dQc[i]  += sum_k dSu[i,k] U[k]  (keys before the pair)  + sum_{j in pair, j <= i} dT[i,j] vu_j
//   dVu[j]  += sum_k A[k,j] G'[k] + sum_{i in pair, i >= j} dT[i,j] qc'_i,   dT[i,j] = sum_k dSu[i,k] A[k,j]
// Head dimensions up to 64: the accumulators of all outputs fit two waves per SIMD (bwd_queryw_kernel
// below is the same kernel laid out for d = 128).
template <typename T, typename TI, int HD>
__global__ __launch_bounds__(2 * kThreads, 2) void bwd_query2_kernel(BwdArgs a) {
  static_assert(sizeof(T) == 2 && kCK == 32 && HD <= 64, "tile consumer: 16-bit operands, d <= 64");
  constexpr int KS = HD / 16;
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr int NT = HDP / 32;
  constexpr int QB = 128;
  constexpr int PT = QB / 32;    // 32-row tiles across the pair
  constexpr int PS = QB / 16;    // 16-deep steps across the pair
  constexpr int LDK = lds_ld_tr<T>(HD), LDT = kLdT2<T>, LDA = kLdA<T>, LDD = kLdD<T>;

  Carver cv{castle_smem};
  T* s_kc = cv.take<T>(kCK * LDK);
  T* s_qu = cv.take<T>(kCK * LDK);
  T* s_ub = cv.take<T>(kCK * LDK);   // lookahead state at the start of the pair
  T* s_g = cv.take<T>(kCK * LDK);    // reverse state behind the pair
  T* s_at = cv.take<T>(QB * LDA);    // gate, [source j][key k]
  T* s_ds = cv.take<T>(kCK * LDD);   // dS,  [key k][query i]
  T* s_dsu = cv.take<T>(kCK * LDD);  // dSu, [key k][query i]
  // the epilogue reuses the same memory
  Carver ce{castle_smem};
  T* e_vu = ce.take<T>(QB * LDK);
  T* e_qc = ce.take<T>(QB * LDK);
  T* e_dt = ce.take<T>(QB * LDT);    // dT, [query i][source j] (pair local)

  int rank, bh;
  work_item(a.s.B * a.s.H, rank, bh);
  const int qb = a.s.Lp / 128 - 1 - rank;   // the last row block meets the most keys
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const bool source_role = wave < 4;
  const int pw = wave & 3;
  const int tid = threadIdx.x & (kThreads - 1);   // thread index inside the role
  const int L = a.s.L;
  const float c0 = a.s.scale, c1 = a.s.scale * kLog2e;
  const float gun = a.bhdr->grad_unscale, vu_scale = a.ws.hdr->vu_scale;
  const int jw = 32 * pw;                     // rows of this wave pair inside the 128-row exchange tiles
  const int i0w = qb * QB + jw;
  const int i = i0w + c;                      // this lane's row
  const int blk0 = 2 * qb, blk1 = 2 * qb + 1;
  const int sfirst = jw / 16;                 // first step covering queries i >= j
  const bool has_g = blk1 <= a.s.nblk - 2;    // a reverse state exists behind the pair

  const T* qc = prep_ptr<T>(a.ws.qc_p, bh, a.s.Lp, HD);
  const T* vu = prep_ptr<T>(a.ws.vu_p, bh, a.s.Lp, HD);
  const T* usnap = reinterpret_cast<const T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  const T* gsnap = reinterpret_cast<const T*>(a.gsnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  const T* ttb = reinterpret_cast<const T*>(a.ws.tt_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* ttx = reinterpret_cast<const T*>(a.ws.ttx_blk) + (int64_t)bh * a.s.Lp * kNB;
  const int64_t tile_row = (int64_t)(a.s.Lp / 32) * 1024;   // elements between the tiles of consecutive key groups
  const T* dsm = reinterpret_cast<const T*>(a.ds_mat) + (int64_t)bh * a.s.Lp * a.s.Lp + (int64_t)qb * 4 * 1024;
  const T* dsum = reinterpret_cast<const T*>(a.dsu_mat) + (int64_t)bh * a.s.Lp * a.s.Lp + (int64_t)qb * 4 * 1024;
  int kend = qb * QB + QB;
  if (kend > a.s.Lp) kend = a.s.Lp;
  TileStage<T, false> pds, pdsu;   // every thread: one piece of each

  if (source_role) {
    const T* kc = prep_ptr<T>(a.ws.kc_p, bh, a.s.Lp, HD);
    const T* qu = prep_ptr<T>(a.ws.qu_p, bh, a.s.Lp, HD);
    const T* ku = prep_ptr<T>(a.ws.ku_p, bh, a.s.Lp, HD);
    // T'^T rows of this wave across the queries of the pair: its own block from tt_blk, and for a
    // wave of the first block the second block from the cross quarter
    frag<T> fku[KS], fvu[KS], ftt[PS];
#pragma unroll
    for (int s = 0; s < KS; ++s) fku[s] = ldg_nat_scaled<T, T>(ku, HD, i, 16 * s + 8 * g, true, -c1);
#pragma unroll
    for (int s = 0; s < KS; ++s) fvu[s] = ldg_nat<T>(vu, HD, i, 16 * s + 8 * g, true);
#pragma unroll
    for (int s = 0; s < PS; ++s) {
      const bool own = (s < PS / 2) == (pw < 2);   // queries of step s lie in this wave's own block
      const T* src = own ? ttb : ttx;
      ftt[s] = ldg_nat<T>(src, kNB, i, 16 * (s % (PS / 2)) + 8 * g, s >= sfirst);
    }
    acc_t dku[NT];   // [n rows, j lanes]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero(dku[nt]);

    // this role stages kc, qu and the lookahead state
    RowStage<T, T, kCK, HD> pkc, pqu;
    SnapStage<T, kCK, HD> pu;
#define CASTLE_BQ2_LOAD_A(K0)                                                            \
  do {                                                                                   \
    pkc.load_flat(kc + (int64_t)(K0) * HD, tid);                                         \
    pqu.load_flat(qu + (int64_t)(K0) * HD, tid);                                         \
    if ((K0) / kNB < blk0) pu.load(usnap + (usnap_off(blk0) + (K0)) * HD, tid);          \
    pds.load(dsm + (int64_t)((K0) / 32) * tile_row);                                     \
    pdsu.load(dsum + (int64_t)((K0) / 32) * tile_row);                                   \
  } while (0)
    CASTLE_BQ2_LOAD_A(0);
    for (int k0 = 0; k0 < kend; k0 += kCK) {
      const int Kb = k0 / kNB;
      __syncthreads();   // 1: tiles free
      pkc.store(s_kc, LDK, tid);
      pqu.store(s_qu, LDK, tid);
      if (Kb < blk0) pu.store(s_ub, LDK, tid);
      pds.store(s_ds);
      pdsu.store(s_dsu);
      if (k0 + kCK < kend) CASTLE_BQ2_LOAD_A(k0 + kCK);   // in flight while this chunk is processed
      __syncthreads();   // 2: tiles staged
      const bool live = k0 <= i0w;   // the chunk's keys do not lie beyond this wave's rows
      // gate tile A[k rows, j lanes] for this wave's 32 source rows, shared as A^T[j][k]
      acc_t aK;
      zero(aK);   // a constant operand of the first product where the chunk is live, registers of zeros where it is not
      if (live) {
        zero(aK);
#pragma unroll
        for (int s0 = 0; s0 < KS; s0 += 4) {   // operand fragments in batches of four
          frag<T> oqu[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) oqu[u] = ld_nat<T>(s_qu, LDK, c, 16 * (s0 + u) + 8 * g);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (s0 + u < KS) mma(aK, oqu[u], fku[s0 + u]);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) aK[r] = fast_rcp(1.f + fast_exp2(aK[r]));
        if (k0 + 31 >= i0w) {   // the tile reaches the diagonal: keep j > k only
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (i <= k0 + acc_row(r, g)) aK[r] = 0.f;
        }
      }
      // a wave the chunk has passed still owes zeros: the later rows of the pair read its rows
#pragma unroll
      for (int q = 0; q < 4; ++q) st4<T>(s_at + (jw + c) * LDA + 8 * q + 4 * g, pack4<T>(aK, q));
      __syncthreads();   // 3: gate shared
      if (!live) continue;
      // dA in two accumulators (two dependent MFMA chains instead of one of up to twelve)
      acc_t dA, dA2;
      zero(dA);
      zero(dA2);
      frag<T> og[KS];
#pragma unroll
      for (int s = 0; s < KS; ++s) og[s] = has_g ? ld_nat<T>(s_g, LDK, c, 16 * s + 8 * g) : zero_frag<T>();
#pragma unroll
      for (int half = 0; half < 2; ++half) {   // two batches keep the operand fragments in registers
        frag<T> ods[PS / 2];
#pragma unroll
        for (int u = 0; u < PS / 2; ++u) ods[u] = ld_nat<T>(s_dsu, LDD, c, 16 * (PS - 1 - (half * (PS / 2) + u)) + 8 * g);
        __builtin_amdgcn_sched_barrier(0);
        // steps from the last one down: the last two run for every wave, so the product that starts
        // dA is unconditional and takes the zero as a constant operand
#pragma unroll
        for (int u = 0; u < PS / 2; ++u) {
          const int step = PS - 1 - (half * (PS / 2) + u);
          if (step >= PS - 2 || step >= sfirst) mma(dA, ods[u], ftt[step]);
          if (half == 0 && u < KS) mma(dA2, og[u], fvu[u]);   // og is zero where no reverse state exists
        }
      }
      acc_t dz;
#pragma unroll
      for (int r = 0; r < 16; ++r) dz[r] = (dA[r] + dA2[r]) * __builtin_fmaf(-aK[r], aK[r], aK[r]);   // A (1 - A) in one instruction
      {
        frag<T> oqt[2][NT];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) oqt[u][nt] = ld_free<T, true>(s_qu, LDK, 32 * nt, HD, 16 * u, c, g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const frag<T> fdz = chain<T>(dz, u);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) mma(dku[nt], oqt[u][nt], fdz);
        }
      }
    }
#undef CASTLE_BQ2_LOAD_A
    // ---- epilogue (the other role's): only the shared staging ---------------------------------
    __syncthreads();   // e1: chunk tiles dead
    {
      RowStage<T, T, QB, HD, 2 * kThreads> st;
      st.load_flat(vu + (int64_t)qb * QB * HD); st.store(e_vu, LDK);
      st.load_flat(qc + (int64_t)qb * QB * HD); st.store(e_qc, LDK);
    }
    __syncthreads();   // e2: epilogue tiles and dT shared
    if (i < L) store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dku, b, h) + (int64_t)i * a.dku.sl, dku, c0 * kLn2 * gun, g, a.s.rotary ? i : -1);
  } else {
    acc_t dqc[NT];   // [n rows, i lanes]
    acc_t dvu[NT];   // [n rows, j lanes]: this role's rows taken as lookahead sources
    acc_t dtacc[PT];            // [j rows (pair local), i lanes]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero(dqc[nt]);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero(dvu[nt]);
#pragma unroll
    for (int jt = 0; jt < PT; ++jt) zero(dtacc[jt]);
    // this role stages the reverse state
    SnapStage<T, kCK, HD> pg;
#define CASTLE_BQ2_LOAD_B(K0)                                                                             \
  do {                                                                                                    \
    if (has_g) pg.load(gsnap + (gsnap_off(blk1) + (K0)) * HD, tid);                                       \
    pds.load(dsm + (int64_t)((K0) / 32) * tile_row);                                                      \
    pdsu.load(dsum + (int64_t)((K0) / 32) * tile_row);                                                    \
  } while (0)
    CASTLE_BQ2_LOAD_B(0);
    for (int k0 = 0; k0 < kend; k0 += kCK) {
      const int Kb = k0 / kNB;
      __syncthreads();   // 1
      if (has_g) pg.store(s_g, LDK, tid);
      pds.store(s_ds);
      pdsu.store(s_dsu);
      if (k0 + kCK < kend) CASTLE_BQ2_LOAD_B(k0 + kCK);
      __syncthreads();   // 2
      const bool live = k0 <= i0w;
      frag<T> bdsu[2];
      if (live) {
        frag<T> bds[2], okt[2][NT], out[2][NT];   // the operand fragments of both 16-key steps are requested together
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          bdsu[s2] = ld_free<T, false>(s_dsu, LDD, jw, 1 << 30, 16 * s2, c, g);
          bds[s2] = ld_free<T, false>(s_ds, LDD, jw, 1 << 30, 16 * s2, c, g);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            okt[s2][nt] = ld_free<T, false>(s_kc, LDK, 32 * nt, HD, 16 * s2, c, g);
            out[s2][nt] = ld_free<T, false>(s_ub, LDK, 32 * nt, HD, 16 * s2, c, g);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            mma(dqc[nt], okt[s2][nt], bds[s2]);
            if (Kb < blk0) mma(dqc[nt], out[s2][nt], bdsu[s2]);
          }
      }
      __syncthreads();   // 3
      if (!live) continue;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {   // one 16-key step at a time keeps the operand registers few
        frag<T> oat[PT], ogt[NT];
#pragma unroll
        for (int jt = 0; jt < PT; ++jt)
          if (jt <= pw) oat[jt] = ld_nat<T>(s_at, LDA, 32 * jt + c, 16 * s2 + 8 * g);
        // dVu += G'^T A for the rows taken as sources: A^T[j][k] of this wave's own rows
        const frag<T> fa = ld_nat<T>(s_at, LDA, jw + c, 16 * s2 + 8 * g);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          ogt[nt] = has_g ? ld_free<T, false>(s_g, LDK, 32 * nt, HD, 16 * s2, c, g) : zero_frag<T>();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jt = 0; jt < PT; ++jt)
          if (jt <= pw) mma(dtacc[jt], oat[jt], bdsu[s2]);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) mma(dvu[nt], ogt[nt], fa);   // ogt is zero where no reverse state exists
      }
    }
#undef CASTLE_BQ2_LOAD_B
    // ---- epilogue: dT = tril(dTacc) over the pair:  dqc += dT Vu,  dvu += dT^T Qc' ------------
    __syncthreads();   // e1
    {
      RowStage<T, T, QB, HD, 2 * kThreads> st;
      st.load_flat(vu + (int64_t)qb * QB * HD); st.store(e_vu, LDK);
      st.load_flat(qc + (int64_t)qb * QB * HD); st.store(e_qc, LDK);
    }
    // dT^T[j rows, i lanes] masked to j <= i, shared as dT[i][j] for the source-side product
#pragma unroll
    for (int jt = 0; jt < PT; ++jt) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (32 * jt + acc_row(r, g) > jw + c) dtacc[jt][r] = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) st4<T>(e_dt + (jw + c) * LDT + 32 * jt + 8 * q + 4 * g, pack4<T>(dtacc[jt], q));
    }
    __syncthreads();   // e2
#pragma unroll
    for (int jt = 0; jt < PT; ++jt) {
      if (jt > pw) continue;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const frag<T> fdt = chain<T>(dtacc[jt], s2);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          mma(dqc[nt], ld_free<T, true>(e_vu, LDK, 32 * nt, HD, 32 * jt + 16 * s2, c, g), fdt);
      }
    }
#pragma unroll
    for (int s = 0; s < PS; ++s) {
      if (s < sfirst) continue;
      // B operand: source j = jw + c on lanes, queries i = 16 s .. in natural order, from dT[i][j]
      const frag<T> fdt = ld_free<T, false>(e_dt, LDT, jw, QB, 16 * s, c, g);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        mma(dvu[nt], ld_free<T, false>(e_qc, LDK, 32 * nt, HD, 16 * s, c, g), fdt);
    }
    if (i < L) {
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dqc, b, h) + (int64_t)i * a.dqc.sl, dqc, c0 * gun, g, a.s.rotary ? i : -1);
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dvu, b, h) + (int64_t)i * a.dvu.sl, dvu, kLn2 * gun * vu_scale, g, a.s.rotary ? i : -1);
    }
  }
}

// ---------------------------------------------------------------------------
// The tile-consuming query-stationary backward for head dimensions above 64, in ONE launch.  Same
// 128 rows per workgroup and same chunks of 32 keys as bwd_query2_kernel, but two barriers per chunk
// (the gate is computed ahead of the second), and the outputs are dealt to the two waves of a pair so that neither holds
// more than half a SIMD's registers:
//   waves 0-3 (source rows j):  gate A, dA, dZ, dKu (all columns), dVu columns 0 .. 31 (the gate
//                               operand of  dVu += G'^T A  comes straight from their registers)
//   waves 4-7 (query rows i):   dQc (all columns), dT, dVu columns 32 .. d - 1
// Every tile, snapshot and gate is read or formed once (two launches with half of the outputs each
// read the dSu tiles, and formed the gate and dT, twice).
template <typename T, int HD> constexpr int bwd_queryw_lds_bytes() {
  int b = 5 * a16((int)sizeof(T) * kCK * lds_ld_tr<T>(HD));       // kc, qu (two chunks), ub, g
  b += a16((int)sizeof(T) * 128 * kLdA<T>);                       // A^T [j][k]
  b += 2 * a16((int)sizeof(T) * kCK * kLdD<T>);                   // dS, dSu [k][i]
  b += a16((int)sizeof(T) * 128 * kLdTT<T>) + a16((int)sizeof(T) * 128 * lds_ld_tr<T>(HD));   // T'^T and vu rows
  int e = 2 * a16((int)sizeof(T) * 128 * lds_ld_tr<T>(HD)) + a16((int)sizeof(T) * 128 * kLdT2<T>);
  return b > e ? b : e;
}

template <typename T, typename TI, int HD>
__global__ __launch_bounds__(2 * kThreads, 2) void bwd_queryw_kernel(BwdArgs a) {
  static_assert(sizeof(T) == 2 && kCK == 32 && HD > 64, "tile consumer for wide heads: 16-bit operands");
  constexpr int KS = HD / 16;
  constexpr int NT = HD / 32;
  constexpr int NHA = 1, NHB = NT - NHA;   // dVu tiles of the source-row / query-row waves (what the registers of each allow)
  constexpr int QB = 128;
  constexpr int PT = QB / 32;    // 32-row tiles across the pair
  constexpr int PS = QB / 16;    // 16-deep steps across the pair
  constexpr int LDK = lds_ld_tr<T>(HD), LDT = kLdT2<T>, LDA = kLdA<T>, LDD = kLdD<T>, LDTT = kLdTT<T>;

  Carver cv{castle_smem};
  T* s_kc = cv.take<T>(kCK * LDK);
  T* s_qu2 = cv.take<T>(2 * kCK * LDK);   // qu rows of a chunk, chunk n in buffer n & 1: staged one chunk ahead (see the source-row waves)
  T* s_ub = cv.take<T>(kCK * LDK);   // lookahead state at the start of the pair
  T* s_g = cv.take<T>(kCK * LDK);    // reverse state behind the pair
  T* s_at = cv.take<T>(QB * LDA);    // gate, [source j][key k]
  T* s_ds = cv.take<T>(kCK * LDD);   // dS,  [key k][query i]
  T* s_dsu = cv.take<T>(kCK * LDD);  // dSu, [key k][query i]
  T* s_tt = cv.take<T>(QB * LDTT);   // T'^T [source j][query i of the pair]
  T* s_vu = cv.take<T>(QB * LDK);    // vu rows of the pair
  // the epilogue reuses the same memory
  Carver ce{castle_smem};
  T* e_vu = ce.take<T>(QB * LDK);
  T* e_qc = ce.take<T>(QB * LDK);
  T* e_dt = ce.take<T>(QB * LDT);    // dT, [query i][source j] (pair local)

  int rank, bh;
  work_item(a.s.B * a.s.H, rank, bh);
  const int qb = a.s.Lp / 128 - 1 - rank;   // the last row block meets the most keys
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const bool source_role = wave < 4;
  const int pw = wave & 3;
  const int tid = threadIdx.x & (kThreads - 1);   // thread index inside the role
  const int L = a.s.L;
  const float c0 = a.s.scale, c1 = a.s.scale * kLog2e;
  const float gun = a.bhdr->grad_unscale, vu_scale = a.ws.hdr->vu_scale;
  const int jw = 32 * pw;                     // rows of this wave pair inside the 128-row exchange tiles
  const int i0w = qb * QB + jw;
  const int i = i0w + c;                      // this lane's row
  const int blk0 = 2 * qb, blk1 = 2 * qb + 1;
  const int sfirst = jw / 16;                 // first step covering queries i >= j
  const bool has_g = blk1 <= a.s.nblk - 2;    // a reverse state exists behind the pair

  const T* qc = prep_ptr<T>(a.ws.qc_p, bh, a.s.Lp, HD);
  const T* vu = prep_ptr<T>(a.ws.vu_p, bh, a.s.Lp, HD);
  const T* usnap = reinterpret_cast<const T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  const T* gsnap = reinterpret_cast<const T*>(a.gsnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;
  const T* ttb = reinterpret_cast<const T*>(a.ws.tt_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* ttx = reinterpret_cast<const T*>(a.ws.ttx_blk) + (int64_t)bh * a.s.Lp * kNB;
  const int64_t tile_row = (int64_t)(a.s.Lp / 32) * 1024;   // elements between the tiles of consecutive key groups
  const T* dsm = reinterpret_cast<const T*>(a.ds_mat) + (int64_t)bh * a.s.Lp * a.s.Lp + (int64_t)qb * 4 * 1024;
  const T* dsum = reinterpret_cast<const T*>(a.dsu_mat) + (int64_t)bh * a.s.Lp * a.s.Lp + (int64_t)qb * 4 * 1024;
  int kend = qb * QB + QB;
  if (kend > a.s.Lp) kend = a.s.Lp;
  TileStage<T, true> pds, pdsu;   // every thread: one piece of each

  {
    // rows j of the pair: T'^T[j][i] over the pair's queries (own block from tt_blk; for the first
    // block the second block's queries from the cross quarter), and vu_j.  Columns a row never
    // uses (queries before its block) are left unwritten.
    constexpr int VH = kNB / 8;   // 16-byte pieces per half row
    for (int p = threadIdx.x; p < QB * 2 * VH; p += 2 * kThreads) {
      const int j = p / (2 * VH), half = (p / VH) & 1, v = p % VH;
      const bool first = j < kNB;
      if (!first && half == 0) continue;
      const T* src = (first && half == 1) ? ttx : ttb;
      *reinterpret_cast<frag_mem<T>*>(s_tt + j * LDTT + half * kNB + v * 8) =
          *reinterpret_cast<const frag_mem<T>*>(src + ((int64_t)qb * QB + j) * kNB + v * 8);
    }
    RowStage<T, T, QB, HD, 2 * kThreads> st;
    st.load_flat(vu + (int64_t)qb * QB * HD);
    st.store(s_vu, LDK);
    // visible after the first barrier of the chunk loop; first used behind its third
  }

  if (source_role) {
    const T* kc = prep_ptr<T>(a.ws.kc_p, bh, a.s.Lp, HD);
    const T* qu = prep_ptr<T>(a.ws.qu_p, bh, a.s.Lp, HD);
    const T* ku = prep_ptr<T>(a.ws.ku_p, bh, a.s.Lp, HD);
    frag<T> fku[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) fku[s] = ldg_nat_scaled<T, T>(ku, HD, i, 16 * s + 8 * g, true, -c1);
    acc_t dku[NT];   // [n rows, j lanes]
    acc_t dvu[NHA];   // [n rows, j lanes], columns 0 .. 31
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero(dku[nt]);
#pragma unroll
    for (int nt = 0; nt < NHA; ++nt) zero(dvu[nt]);

    // This role stages kc, qu and its half of the dS / dSu tiles.  The qu rows run one chunk ahead of the
    // rest (two LDS buffers): the gate of a chunk then needs nothing that is staged in that chunk, and
    // is computed between barriers 1 and 2, while the partner waves are still held up requesting their
    // snapshot rows - two barriers per chunk instead of three, and no wave idles behind barrier 1.
    RowStage<T, T, kCK, HD> pkc, pqu;
#define CASTLE_BQW_LOAD_A(K0)                                                       \
  do {                                                                              \
    pkc.load_flat(kc + (int64_t)(K0) * HD, tid);                                    \
    if ((K0) + kCK < kend) pqu.load_flat(qu + (int64_t)((K0) + kCK) * HD, tid);     \
    pds.load(dsm + (int64_t)((K0) / 32) * tile_row);                                \
    pdsu.load(dsum + (int64_t)((K0) / 32) * tile_row);                              \
  } while (0)
    pqu.load_flat(qu, tid);
    pqu.store(s_qu2, LDK, tid);   // chunk 0: visible behind the first barrier
    CASTLE_BQW_LOAD_A(0);
    for (int k0 = 0; k0 < kend; k0 += kCK) {
      const T* s_qu = s_qu2 + ((k0 / kCK) & 1) * kCK * LDK;
      __syncthreads();   // 1: tiles free
      pkc.store(s_kc, LDK, tid);
      if (k0 + kCK < kend) pqu.store(s_qu2 + (((k0 / kCK) & 1) ^ 1) * kCK * LDK, LDK, tid);
      pds.store(s_ds);
      pdsu.store(s_dsu);
      if (k0 + kCK < kend) CASTLE_BQW_LOAD_A(k0 + kCK);   // in flight while this chunk is processed
      const bool live = k0 <= i0w;   // the chunk's keys do not lie beyond this wave's rows
      // gate tile A[k rows, j lanes] for this wave's 32 source rows, shared as A^T[j][k]
      acc_t aK;
      zero(aK);   // a constant operand of the first product where the chunk is live, registers of zeros where it is not
      if (live) {
        zero(aK);
#pragma unroll
        for (int s0 = 0; s0 < KS; s0 += 4) {   // operand fragments in batches of four
          frag<T> oqu[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) oqu[u] = ld_nat<T>(s_qu, LDK, c, 16 * (s0 + u) + 8 * g);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int u = 0; u < 4; ++u) mma(aK, oqu[u], fku[s0 + u]);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) aK[r] = fast_rcp(1.f + fast_exp2(aK[r]));
        if (k0 + 31 >= i0w) {   // the tile reaches the diagonal: keep j > k only
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (i <= k0 + acc_row(r, g)) aK[r] = 0.f;
        }
      }
      // a wave the chunk has passed still owes zeros: the later rows of the pair read its rows
#pragma unroll
      for (int q = 0; q < 4; ++q) st4<T>(s_at + (jw + c) * LDA + 8 * q + 4 * g, pack4<T>(aK, q));
      __syncthreads();   // 2: tiles staged, gate shared
      if (!live) continue;
      // dA in two accumulators (two dependent MFMA chains instead of one)
      acc_t dA, dA2;
      zero(dA);
      zero(dA2);
#pragma unroll
      for (int s0 = 0; s0 < PS; s0 += 2) {   // dSu^T T' and G' Vu^T, two steps of each at a time
        frag<T> ods[2], ott[2], og[2], ovu[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          ods[u] = ld_nat<T>(s_dsu, LDD, c, 16 * (s0 + u) + 8 * g);
          ott[u] = ld_nat<T>(s_tt, LDTT, jw + c, 16 * (s0 + u) + 8 * g);
          og[u] = has_g ? ld_nat<T>(s_g, LDK, c, 16 * (s0 + u) + 8 * g) : zero_frag<T>();   // zero where no reverse state exists
          ovu[u] = ld_nat<T>(s_vu, LDK, jw + c, 16 * (s0 + u) + 8 * g);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          if (s0 + u >= sfirst) mma(dA, ods[u], ott[u]);
          mma(dA2, og[u], ovu[u]);
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) dA[r] = (dA[r] + dA2[r]) * __builtin_fmaf(-aK[r], aK[r], aK[r]);   // dZ; A (1 - A) in one instruction
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {   // small batches of operand fragments: this role is at the register limit
        const frag<T> fdz = chain<T>(dA, s2), fa = chain<T>(aK, s2);
#pragma unroll
        for (int n0 = 0; n0 < NT; n0 += 2) {
          frag<T> oqt[2];
#pragma unroll
          for (int u = 0; u < 2; ++u) oqt[u] = ld_free<T, true>(s_qu, LDK, 32 * (n0 + u), HD, 16 * s2, c, g);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int u = 0; u < 2; ++u) mma(dku[n0 + u], oqt[u], fdz);
        }
        frag<T> ogt[NHA];
#pragma unroll
        for (int nt = 0; nt < NHA; ++nt) ogt[nt] = has_g ? ld_free<T, true>(s_g, LDK, 32 * nt, HD, 16 * s2, c, g) : zero_frag<T>();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nt = 0; nt < NHA; ++nt) mma(dvu[nt], ogt[nt], fa);   // dVu += G'^T A; ogt is zero where no reverse state exists
      }
    }
#undef CASTLE_BQW_LOAD_A
    // ---- epilogue: dvu += dT^T Qc' for this role's columns ------------------------------------
    __syncthreads();   // e1: chunk tiles dead
    {
      RowStage<T, T, QB, HD, 2 * kThreads> st;
      st.load_flat(vu + (int64_t)qb * QB * HD); st.store(e_vu, LDK);
      st.load_flat(qc + (int64_t)qb * QB * HD); st.store(e_qc, LDK);
    }
    __syncthreads();   // e2: epilogue tiles and dT shared
#pragma unroll
    for (int s = 0; s < PS; ++s) {
      if (s < sfirst) continue;
      // B operand: source j = jw + c on lanes, queries i = 16 s .. in natural order, from dT[i][j]
      const frag<T> fdt = ld_free<T, false>(e_dt, LDT, jw, QB, 16 * s, c, g);
#pragma unroll
      for (int nt = 0; nt < NHA; ++nt)
        mma(dvu[nt], ld_free<T, false>(e_qc, LDK, 32 * nt, HD, 16 * s, c, g), fdt);
    }
    if (i < L) {
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dku, b, h) + (int64_t)i * a.dku.sl, dku, c0 * kLn2 * gun, g, a.s.rotary ? i : -1);
      store_rows<TI, HD, NHA>(head_ptr_mut<TI>(a.dvu, b, h) + (int64_t)i * a.dvu.sl, dvu, kLn2 * gun * vu_scale, g, a.s.rotary ? i : -1, 0);
    }
  } else {
    acc_t dqc[NT];      // [n rows, i lanes]
    acc_t dvu[NHB];      // [n rows, j lanes], columns 32 .. HD - 1: this role's rows taken as lookahead sources
    acc_t dtacc[PT];    // [j rows (pair local), i lanes]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero(dqc[nt]);
#pragma unroll
    for (int nt = 0; nt < NHB; ++nt) zero(dvu[nt]);
#pragma unroll
    for (int jt = 0; jt < PT; ++jt) zero(dtacc[jt]);
    // this role stages the two states and its half of the dS / dSu tiles
    SnapStage<T, kCK, HD> pu, pg;
#define CASTLE_BQW_LOAD_B(K0)                                                          \
  do {                                                                                 \
    if ((K0) / kNB < blk0) pu.load(usnap + (usnap_off(blk0) + (K0)) * HD, tid);        \
    if (has_g) pg.load(gsnap + (gsnap_off(blk1) + (K0)) * HD, tid);                    \
    pds.load(dsm + (int64_t)((K0) / 32) * tile_row);                                   \
    pdsu.load(dsum + (int64_t)((K0) / 32) * tile_row);                                 \
  } while (0)
    CASTLE_BQW_LOAD_B(0);
    for (int k0 = 0; k0 < kend; k0 += kCK) {
      const int Kb = k0 / kNB;
      __syncthreads();   // 1
      if (Kb < blk0) pu.store(s_ub, LDK, tid);
      if (has_g) pg.store(s_g, LDK, tid);
      pds.store(s_ds);
      pdsu.store(s_dsu);
      if (k0 + kCK < kend) CASTLE_BQW_LOAD_B(k0 + kCK);
      __syncthreads();   // 2
      const bool live = k0 <= i0w;
      frag<T> bdsu[2];
      if (live) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {   // one 16-key step at a time keeps the operand registers few
          bdsu[s2] = ld_free<T, false>(s_dsu, LDD, jw, 1 << 30, 16 * s2, c, g);
          const frag<T> bds = ld_free<T, false>(s_ds, LDD, jw, 1 << 30, 16 * s2, c, g);
#pragma unroll
          for (int n0 = 0; n0 < NT; n0 += 2) {
            frag<T> okt[2], out[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
              okt[u] = ld_free<T, false>(s_kc, LDK, 32 * (n0 + u), HD, 16 * s2, c, g);
              out[u] = ld_free<T, false>(s_ub, LDK, 32 * (n0 + u), HD, 16 * s2, c, g);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < 2; ++u) {
              mma(dqc[n0 + u], okt[u], bds);
              if (Kb < blk0) mma(dqc[n0 + u], out[u], bdsu[s2]);
            }
          }
        }
      }
      if (!live) continue;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {   // two small batches of operand fragments: this role is at the register limit
        {
          frag<T> oat[PT];
#pragma unroll
          for (int jt = 0; jt < PT; ++jt)
            if (jt <= pw) oat[jt] = ld_nat<T>(s_at, LDA, 32 * jt + c, 16 * s2 + 8 * g);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int jt = 0; jt < PT; ++jt)
            if (jt <= pw) mma(dtacc[jt], oat[jt], bdsu[s2]);
        }
        __builtin_amdgcn_sched_barrier(0);
        {
          // dVu += G'^T A for the rows taken as sources: A^T[j][k] of this wave's own rows
          frag<T> ogt[NHB];
          const frag<T> fa = ld_nat<T>(s_at, LDA, jw + c, 16 * s2 + 8 * g);
#pragma unroll
          for (int nt = 0; nt < NHB; ++nt)
            ogt[nt] = has_g ? ld_free<T, false>(s_g, LDK, 32 * (NHA + nt), HD, 16 * s2, c, g) : zero_frag<T>();
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int nt = 0; nt < NHB; ++nt) mma(dvu[nt], ogt[nt], fa);   // ogt is zero where no reverse state exists
        }
      }
    }
#undef CASTLE_BQW_LOAD_B
    // ---- epilogue: dT = tril(dTacc) over the pair:  dqc += dT Vu,  dvu += dT^T Qc' ------------
    __syncthreads();   // e1
    {
      RowStage<T, T, QB, HD, 2 * kThreads> st;
      st.load_flat(vu + (int64_t)qb * QB * HD); st.store(e_vu, LDK);
      st.load_flat(qc + (int64_t)qb * QB * HD); st.store(e_qc, LDK);
    }
    // dT^T[j rows, i lanes] masked to j <= i, shared as dT[i][j] for the source-side product
#pragma unroll
    for (int jt = 0; jt < PT; ++jt) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (32 * jt + acc_row(r, g) > jw + c) dtacc[jt][r] = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) st4<T>(e_dt + (jw + c) * LDT + 32 * jt + 8 * q + 4 * g, pack4<T>(dtacc[jt], q));
    }
    __syncthreads();   // e2
#pragma unroll
    for (int jt = 0; jt < PT; ++jt) {
      if (jt > pw) continue;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const frag<T> fdt = chain<T>(dtacc[jt], s2);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          mma(dqc[nt], ld_free<T, true>(e_vu, LDK, 32 * nt, HD, 32 * jt + 16 * s2, c, g), fdt);
      }
    }
#pragma unroll
    for (int s = 0; s < PS; ++s) {
      if (s < sfirst) continue;
      const frag<T> fdt = ld_free<T, false>(e_dt, LDT, jw, QB, 16 * s, c, g);
#pragma unroll
      for (int nt = 0; nt < NHB; ++nt)
        mma(dvu[nt], ld_free<T, false>(e_qc, LDK, 32 * (NHA + nt), HD, 16 * s, c, g), fdt);
    }
    if (i < L) {
      store_rows<TI, HD, NT>(head_ptr_mut<TI>(a.dqc, b, h) + (int64_t)i * a.dqc.sl, dqc, c0 * gun, g, a.s.rotary ? i : -1);
      store_rows<TI, HD, NHB>(head_ptr_mut<TI>(a.dvu, b, h) + (int64_t)i * a.dvu.sl, dvu, kLn2 * gun * vu_scale, g, a.s.rotary ? i : -1, NHA);
    }
  }
}

// ---------------------------------------------------------------------------
// raises the dynamic-LDS limit of the single-role kernels (once per device); launches nothing
template <typename T, typename TI, int HD, int PART> static int configure_single_role_kernels() {
  constexpr int key_lds = bwd_key_lds_bytes<T, HD>(), query_lds = bwd_query_lds_bytes<T, HD>();
  static PerDeviceOnce once;
  bool& configured = once.flag();
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_key_kernel<T, TI, HD, PART>), hipFuncAttributeMaxDynamicSharedMemorySize, key_lds) != hipSuccess) return -3;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_query_kernel<T, TI, HD, PART>), hipFuncAttributeMaxDynamicSharedMemorySize, query_lds) != hipSuccess) return -3;
    configured = true;
  }
  return 0;
}

template <typename T, typename TI, int HD> static int launch_bwd_t(const BwdArgs& a, hipStream_t stream) {
  const int BH = a.s.B * a.s.H;
  constexpr int key_lds = bwd_key_lds_bytes<T, HD>(), query_lds = bwd_query_lds_bytes<T, HD>();
  if (key_lds > kMaxLds || query_lds > kMaxLds) return -2;
  constexpr bool SPLIT = HD > 64;   // two passes per kernel, half of the outputs each
  constexpr bool TWO_ROLE = sizeof(T) == 2 && HD <= 64;
  constexpr bool TILES = sizeof(T) == 2;   // the query-stationary kernel can read dS / dSu tiles
  if constexpr (TWO_ROLE) {
    static PerDeviceOnce once2;
    bool& configured2 = once2.flag();
    if (!configured2) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_key2_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, bwd_key2_lds_bytes<T, HD>()) != hipSuccess) return -3;
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_query2_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, bwd_query2_lds_bytes<T, HD>()) != hipSuccess) return -3;
      configured2 = true;
    }
  } else if constexpr (TILES) {   // 16-bit tensors at d = 128: the two-role kernels for wide heads
    static_assert(bwd_queryw_lds_bytes<T, HD>() <= kMaxLds, "wide-head query kernel does not fit the LDS");
    static_assert(bwd_keyw1_lds_bytes<T, HD>() <= kMaxLds && bwd_keyw2_lds_bytes<T, HD>() <= kMaxLds, "wide-head key kernels do not fit the LDS");
    static PerDeviceOnce once3;
    bool& configured3 = once3.flag();
    if (!configured3) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_queryw_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, bwd_queryw_lds_bytes<T, HD>()) != hipSuccess) return -3;
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_keyw1_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, bwd_keyw1_lds_bytes<T, HD>()) != hipSuccess) return -3;
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_keyw2_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, bwd_keyw2_lds_bytes<T, HD>()) != hipSuccess) return -3;
      configured3 = true;
    }
  }
  int rc = 0;
  if constexpr (SPLIT) {
    rc = configure_single_role_kernels<T, TI, HD, 1>();
    if (rc == 0) rc = configure_single_role_kernels<T, TI, HD, 2>();
  } else {
    rc = configure_single_role_kernels<T, TI, HD, 0>();
  }
  if (rc != 0) return rc;
  constexpr int RPB = kThreads / (HD / elem_traits<T>::vec16);
  const dim3 grid(a.s.Lp / 128 * BH), block(kThreads);
  {
    ProfScope ps(kSlotDelta, stream);
    if constexpr (sizeof(T) == 2)
      hipLaunchKernelGGL((amax_kernel<TI, HD>), dim3(kAmaxBlocks), dim3(kAmaxThreads), 0, stream, a.dout, a.s.H, a.s.L,
                         (int64_t)BH * a.s.L, a.amax_part, (int*)nullptr);
    hipLaunchKernelGGL((delta_kernel<T, TI, HD>), dim3((a.s.Lp + RPB - 1) / RPB, BH), block, 0, stream, a);
  }
  {
    ProfScope ps(kSlotBwdKey, stream);
    if constexpr (SPLIT) {
      bool from_tiles = false;
      if constexpr (TILES) {
        if (a.ds_mat != nullptr) {   // room for the dS / dSu tiles: the two-role launches
          constexpr int w1_lds = bwd_keyw1_lds_bytes<T, HD>(), w2_lds = bwd_keyw2_lds_bytes<T, HD>();
          hipLaunchKernelGGL((bwd_keyw1_kernel<T, TI, HD>), grid, dim3(2 * kThreads), w1_lds, stream, a);
          hipLaunchKernelGGL((bwd_keyw2_kernel<T, TI, HD>), grid, dim3(2 * kThreads), w2_lds, stream, a);
          from_tiles = true;
        }
      }
      if (!from_tiles) {
        hipLaunchKernelGGL((bwd_key_kernel<T, TI, HD, 1>), grid, block, key_lds, stream, a);
        hipLaunchKernelGGL((bwd_key_kernel<T, TI, HD, 2>), grid, block, key_lds, stream, a);
      }
    } else if constexpr (TWO_ROLE) {
      constexpr int key2_lds = bwd_key2_lds_bytes<T, HD>();
      hipLaunchKernelGGL((bwd_key2_kernel<T, TI, HD>), grid, dim3(2 * kThreads), key2_lds, stream, a);
    } else {
      hipLaunchKernelGGL((bwd_key_kernel<T, TI, HD, 0>), grid, block, key_lds, stream, a);
    }
  }
  {
    ProfScope ps(kSlotBwdQuery, stream);
    bool done = false;
    if constexpr (TILES) {
      if (a.ds_mat != nullptr) {   // the key kernel left the dS / dSu tiles
        if constexpr (SPLIT) {
          constexpr int queryw_lds = bwd_queryw_lds_bytes<T, HD>();
          hipLaunchKernelGGL((bwd_queryw_kernel<T, TI, HD>), grid, dim3(2 * kThreads), queryw_lds, stream, a);
        } else {
          constexpr int query2_lds = bwd_query2_lds_bytes<T, HD>();
          hipLaunchKernelGGL((bwd_query2_kernel<T, TI, HD>), grid, dim3(2 * kThreads), query2_lds, stream, a);
        }
        done = true;
      }
    }
    if (!done) {   // fp32, or no room for the tiles (long sequences): the recomputing kernel
      if constexpr (SPLIT) {
        hipLaunchKernelGGL((bwd_query_kernel<T, TI, HD, 1>), grid, block, query_lds, stream, a);
        hipLaunchKernelGGL((bwd_query_kernel<T, TI, HD, 2>), grid, block, query_lds, stream, a);
      } else {
        hipLaunchKernelGGL((bwd_query_kernel<T, TI, HD, 0>), grid, block, query_lds, stream, a);
      }
    }
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <typename T, typename TI> static int launch_bwd_d(const BwdArgs& a, hipStream_t stream) {
  switch (a.s.d) {
    case 16: return launch_bwd_t<T, TI, 16>(a, stream);
    case 32: return launch_bwd_t<T, TI, 32>(a, stream);
    case 64: return launch_bwd_t<T, TI, 64>(a, stream);
    case 128:
      if constexpr (sizeof(T) == 2) return launch_bwd_t<T, TI, 128>(a, stream);
      return -2;
    default: return -2;
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
