// CASTLE parallel forward for gfx950: O(L^2 d) state form in three kernels.
//
//   prep_kernel  the six operands -> compute type, [B*H][Lp][d] contiguous, rows >= L zero, Qc
//                pre-multiplied by scale*log2(e); every other kernel reads these copies, so its
//                tile loads need neither conversions nor bounds nor strides
//   tqv_block    per 64-row block I:  T_II = tril(Qc_I Vu_I^T), both orientations, and the cross quarter
//                of a block pair; run by the trailing workgroups of the scan launch
//   scan_kernel  key-stationary: for a group of 128 keys sweep the source blocks I,
//                A_KI = sigmoid(s Qu_K Ku_I^T) (strictly j>k), state += A_KI Vu_I.
//                The state as of the start of block I is stored as snapshot
//                usnap[I][k]; the final state is the cache tensor U.
//   attn_kernel  query-stationary: 128 queries per workgroup (two 64-row blocks),
//                keys streamed in chunks of 64 or 32:
//                  Su = Qc_I usnap[I][K]^T + T_II A_KI^T,  S = s(Sc - Su sigmoid(s Su)),
//                online softmax over keys, O = P Vc.
// The math follows the dense definition at lookahead_keys_attention.py:132-164 of the
// reference.  The softmax scale (times log2 e) is folded once into the operand fragments each
// wave keeps in registers; K/V/state operands stay unscaled.
#include "castle_tiles.h"
#include "castle_params.h"
#include "castle_profile.h"

namespace castle {

extern __shared__ __attribute__((aligned(16))) unsigned char castle_smem[];

// Units.  With c1 = scale * log2(e) the kernels work on "log2-domain" scores:
//   Qc' = c1 Qc            so that  Sc' = Qc' Kc^T        = c1 * (Qc Kc^T)
//   T'  = tril(Qc' Vu^T)   so that  Su' = Qc' U^T + T' A^T = log2(e) * Su
//   gate operand (Qu or Ku, whichever is resident) is multiplied by -c1, so that
//   A = 1 / (1 + exp2(acc)) needs no multiply.
// Then sigmoid(Su) = 1/(1+exp2(-Su')), S' = Sc' - Su' sigmoid(Su) = log2(e) S, P = exp2(S' - m').
// value tile of the scan / attention kernels: 16-bit operands keep it row-major and read it with
// transpose loads, fp32 stores it transposed
template <typename T, int HD> constexpr int vtile_elems() {
  return sizeof(T) == 2 ? kNB * lds_ld_tr<T>(HD) : (HD < 32 ? 32 : HD) * lds_ld_chain<T>(kNB);
}
template <typename T, int HD> constexpr int scan_lds_bytes() {
  return (int)sizeof(T) * (kNB * lds_ld_tr<T>(HD) + vtile_elems<T, HD>());
}
// keys per chunk of the attention kernel: 32 for 16-bit operands from d = 64 up.  At d = 128 the smaller
// tiles and staging registers are what lets two workgroups share a CU (two waves per SIMD instead of
// one: 5.6 -> 3.8 ms at 16 heads x 16384 tokens); at d = 64 they are worth 1.5 %.
template <typename T, int HD> constexpr int attn_chunk() { return sizeof(T) == 2 && HD >= 64 ? 32 : kNB; }
// at d = 128 the T' rows of a wave live in LDS instead of registers (each lane reads back what it wrote)
template <typename T, int HD> constexpr bool attn_t_in_lds() { return sizeof(T) == 2 && HD == 128; }
template <typename T, int HD> constexpr int attn_lds_bytes() {
  constexpr int CK = attn_chunk<T, HD>();
  return (int)sizeof(T) * (4 * CK * lds_ld_tr<T>(HD) + (sizeof(T) == 2 ? CK * lds_ld_tr<T>(HD) : vtile_elems<T, HD>()) + CK * lds_ld<T>(128) +
                           (attn_t_in_lds<T, HD>() ? 128 * lds_ld<T>(kNB) : 0));
}
// register prefetch of the next tile is affordable for 16-bit operands up to d = 64
template <typename T, int HD> constexpr bool use_prefetch() { return sizeof(T) == 2; }

template <typename T> __device__ __forceinline__ const T* head_ptr(const View4& v, int b, int h) {
  return reinterpret_cast<const T*>(v.ptr) + (int64_t)b * v.sb + (int64_t)h * v.sh;
}
template <typename T> __device__ __forceinline__ T* head_ptr_mut(const View4& v, int b, int h) {
  return reinterpret_cast<T*>(v.ptr) + (int64_t)b * v.sb + (int64_t)h * v.sh;
}

// ---------------------------------------------------------------------------
// One 16-byte piece of one operand per thread; blockIdx.z selects the operand.
template <typename T, typename TI, int HD>
__global__ __launch_bounds__(kThreads) void prep_kernel(FwdArgs a) {
  constexpr int V = elem_traits<T>::vec16;
  constexpr int VPR = HD / V;
  const int bh = blockIdx.y, b = bh / a.s.H, h = bh % a.s.H;
  const int64_t piece = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int64_t row = piece / VPR;
  const int cv = (int)(piece % VPR);
  if (row >= a.s.Lp) return;
  View4 src;
  void* dstv;
  float mul = 1.f;
  switch (blockIdx.z) {
    case 0: src = a.qc; dstv = a.ws.qc_p; mul = a.s.scale * kLog2e; break;
    case 1: src = a.kc; dstv = a.ws.kc_p; break;
    case 2: src = a.vc; dstv = a.ws.vc_p; break;
    case 3: src = a.qu; dstv = a.ws.qu_p; break;
    case 4: src = a.ku; dstv = a.ws.ku_p; break;
    default: src = a.vu; dstv = a.ws.vu_p; break;
  }
  if constexpr (sizeof(T) == 2) {
    if (blockIdx.z == 5) {   // vu is brought into the range that keeps every lookahead state finite in fp16
      mul = vu_scale_for(amax_from_partials(a.ws.amax_part), a.s.L);
      if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
        a.ws.hdr->vu_scale = mul;
        a.ws.hdr->su_mul = 1.f / mul;
      }
    }
  } else {
    if (blockIdx.z == 5 && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
      a.ws.hdr->status = 0;
      a.ws.hdr->vu_scale = 1.f;
      a.ws.hdr->su_mul = 1.f;
    }
  }
  vec<float, V> f;
#pragma unroll
  for (int e = 0; e < V; ++e) f[e] = 0.f;
  if (row < a.s.L)
    f = __builtin_convertvector(*reinterpret_cast<const vec<TI, V>*>(head_ptr<TI>(src, b, h) + row * src.sl + cv * V), vec<float, V>);
  if (a.s.rotary && blockIdx.z != 2) {   // every operand but Vc is rotated by its position
#pragma unroll
    for (int e = 0; e < V / 2; ++e) CASTLE_ROPE_PAIR(f[2 * e], f[2 * e + 1], (float)row, cv * (V / 2) + e, HD, false);
  }
#pragma unroll
  for (int e = 0; e < V; ++e) f[e] *= mul;
  if constexpr (__is_same(T, fp16_t) && !__is_same(TI, fp16_t)) {
    // wider input type: values beyond the fp16 range are clamped (and reported in the header)
    bool clamped = false;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const float y = __builtin_amdgcn_fmed3f(f[e], -kHalfMax, kHalfMax);
      clamped |= y != f[e] && f[e] == f[e];
      f[e] = y;
    }
    if (clamped) atomicOr(&a.ws.hdr->status, 1);
  }
  T* dst = reinterpret_cast<T*>(dstv) + ((int64_t)bh * a.s.Lp + row) * HD + cv * V;
  *reinterpret_cast<vec<T, V>*>(dst) = __builtin_convertvector(f, vec<T, V>);
}

// ---------------------------------------------------------------------------
// T' of one 64-row block, by the four waves of a workgroup (one 32x32 tile each).  These blocks have
// no kernel of their own: they are the last workgroups of the scan launch, which reads none of them,
// so they run in the slots the scan's tail leaves empty (its last fifth runs at under half occupancy:
// the launch cannot end before the 64-block sweep of key group 0 does).
template <typename T, typename TI, int HD>
__device__ __forceinline__ void tqv_block(const FwdArgs& a, int I, int bh) {
  constexpr int KS = HD / 16;
  constexpr int TB = kNB / 32;
  static_assert(TB * TB == kThreads / 64, "one 32x32 tile of the block per wave");
  const int lane = lane_id(), c = lane & 31, g = lane >> 5;
  const T* qc = prep_ptr<T>(a.ws.qc_p, bh, a.s.Lp, HD);   // pre-scaled by c1
  const T* vu = prep_ptr<T>(a.ws.vu_p, bh, a.s.Lp, HD);
  T* tb = reinterpret_cast<T*>(a.ws.t_blk) + (int64_t)bh * a.s.Lp * kNB;
  T* ttb = reinterpret_cast<T*>(a.ws.tt_blk) + (int64_t)bh * a.s.Lp * kNB;
  T* ttx = reinterpret_cast<T*>(a.ws.ttx_blk) + (int64_t)bh * a.s.Lp * kNB;
  const int it = wave_id() / TB, jt = wave_id() % TB;
  const int64_t i = (int64_t)I * kNB + 32 * it + c;   // A-operand row
  const int64_t j = (int64_t)I * kNB + 32 * jt + c;   // B-operand row
  // cross quarter of a pair of blocks, (Qc'_{I+1} Vu_I^T)^T for even I: same sources, the queries
  // of the next block, no mask (every query is later).  All operand loads are issued together.
  const bool cross = (I & 1) == 0 && I + 1 < a.s.nblk;
  frag<T> fq[KS], fv[KS], fx[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    fq[s] = ldg_nat<T>(qc, HD, i, 16 * s + 8 * g, true);
    fv[s] = ldg_nat<T>(vu, HD, j, 16 * s + 8 * g, true);
    fx[s] = ldg_nat<T>(qc, HD, i + kNB, 16 * s + 8 * g, cross);
  }
  acc_t acc, accx;
  zero(acc);
  zero(accx);
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    mma(acc, fq[s], fv[s]);
    mma(accx, fx[s], fv[s]);
  }
  if constexpr (__is_same(T, fp16_t)) {   // T' beyond the fp16 range is clamped (and reported in the header)
    bool clamped = false;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float y = __builtin_amdgcn_fmed3f(acc[r], -kHalfMax, kHalfMax), yx = __builtin_amdgcn_fmed3f(accx[r], -kHalfMax, kHalfMax);
      clamped |= (y != acc[r] && acc[r] == acc[r]) || (yx != accx[r] && accx[r] == accx[r]);
      acc[r] = y;
      accx[r] = yx;
    }
    if (clamped) atomicOr(&a.ws.hdr->status, 2);
  }
  // acc[r] = (Qc' Vu^T)[il = 32 it + acc_row][jl = 32 jt + c]; stored as T' = tril(.)
  const int jl = 32 * jt + c;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int il = 32 * it + acc_row(r, g);
    acc[r] = jl > il ? 0.f : acc[r];
    tb[((int64_t)I * kNB + il) * kNB + jl] = (T)acc[r];
  }
#pragma unroll
  for (int q = 0; q < 4; ++q)
    st4<T>(ttb + ((int64_t)I * kNB + jl) * kNB + 32 * it + 8 * q + 4 * g, pack4<T>(acc, q));
  if (cross) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      st4<T>(ttx + ((int64_t)I * kNB + jl) * kNB + 32 * it + 8 * q + 4 * g, pack4<T>(accx, q));
  }
}

// ---------------------------------------------------------------------------
// Waves per SIMD the scan is compiled for (a workgroup is one wave per SIMD).  Stating it matters
// beyond occupancy: a kernel that may take more than 256 registers per lane gets its MFMA
// accumulators in the accumulation-register file, and the compiler then copies the state tiles
// between the two files around every matrix instruction (80 copies per 32x32 gate tile, as many
// instructions as the element-wise work itself: 0.160 -> 0.138 ms at B4 H8 L4096 d64).
template <typename T, int HD> constexpr int scan_waves_per_simd() {
  return sizeof(T) == 2 ? (HD <= 32 ? 5 : HD == 64 ? 3 : 2) : (HD <= 32 ? 4 : HD == 64 ? 3 : 1);
}

template <typename T, typename TI, int HD>
__global__ __launch_bounds__(kThreads, (scan_waves_per_simd<T, HD>())) void scan_kernel(FwdArgs a) {
  constexpr int KS = HD / 16;
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr int NT = HDP / 32;
  constexpr int JT = kNB / 32;
  constexpr int LDK = lds_ld_tr<T>(HD), LDV = lds_ld_chain<T>(kNB);
  constexpr bool PF = use_prefetch<T, HD>();
  T* s_ku = reinterpret_cast<T*>(castle_smem);   // [kNB][LDK]
  T* s_vut = s_ku + kNB * LDK;                   // fp32: [HDP][LDV] (transposed); 16-bit: [kNB][LDK]
  constexpr bool TRV = sizeof(T) == 2;

  {
    const int BH = a.s.B * a.s.H, n_scan = a.s.Lp / 128 * BH;
    if ((int)blockIdx.x >= n_scan) {   // behind the key groups: the T' blocks
      const int id = blockIdx.x - n_scan;
      tqv_block<T, TI, HD>(a, id / BH, id % BH);
      return;
    }
  }
  int kb, bh;   // key group 0 sweeps every source block: rank order = kb
  work_item(a.s.B * a.s.H, kb, bh);
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const int L = a.s.L;
  const float c1 = a.s.scale * kLog2e;
  const int kw0 = kb * 128 + 32 * wave;
  const int k = kw0 + c;
  const T* qu = prep_ptr<T>(a.ws.qu_p, bh, a.s.Lp, HD);
  const T* ku = prep_ptr<T>(a.ws.ku_p, bh, a.s.Lp, HD);
  const T* vu = prep_ptr<T>(a.ws.vu_p, bh, a.s.Lp, HD);
  T* snap = reinterpret_cast<T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;

  frag<T> fq[KS];   // -c1 * Qu rows of this wave
#pragma unroll
  for (int s = 0; s < KS; ++s) fq[s] = ldg_nat_scaled<T, T>(qu, HD, k, 16 * s + 8 * g, true, -c1);
  acc_t st[NT];   // state^T : rows n (head dim), columns k (lanes)
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) zero(st[nt]);
  if (!TRV && HDP > HD) lds_zero(s_vut + HD * LDV, (HDP - HD) * LDV);

#pragma unroll
  for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(fq[s]));   // loaded before the prefetches start
  RowStage<T, T, kNB, HD> pku, pvr;
  ColStage<T, T, kNB, HD> pvu;
  auto load_block = [&](int I) __attribute__((always_inline)) {
    pku.load_flat(ku + (int64_t)I * kNB * HD);
    if (TRV) pvr.load_flat(vu + (int64_t)I * kNB * HD);
    else pvu.load(vu, HD, (int64_t)I * kNB, kNoRowLimit);
  };
  const int I0 = (kb * 128) / kNB;
  if (PF) load_block(I0);
  for (int I = I0; I < a.s.nblk; ++I) {
    __syncthreads();
    if (!PF) load_block(I);
    pku.store(s_ku, LDK);
    if (TRV) pvr.store(s_vut, LDK);
    else pvu.store(s_vut, LDV);
    // after the staging wait, not before it: the wait counter also covers stores, and these
    // then have the whole block to drain
    if (I * kNB >= kw0 + 32) {   // all keys of this wave precede block I: snapshot
      store_snap_tile<T, HD, NT>(snap + (usnap_off(I) + kw0) * HD, st, c, g);
    }
    if (PF && I + 1 < a.s.nblk) load_block(I + 1);   // in flight while this block is processed
    __syncthreads();
#pragma unroll
    for (int jt = 0; jt < JT; ++jt) {
      const int j0 = I * kNB + 32 * jt;
      if (j0 + 31 <= kw0) continue;   // every j <= every k of this wave
      acc_t aT;                       // A^T tile: rows j, columns k
      zero(aT);
#pragma unroll
      for (int s = 0; s < KS; ++s) mma(aT, ld_nat<T>(s_ku, LDK, 32 * jt + c, 16 * s + 8 * g), fq[s]);
#pragma unroll
      for (int r = 0; r < 16; ++r) aT[r] = fast_rcp(1.f + fast_exp2(aT[r]));
      if (j0 <= kw0 + 31) {           // tile touches the diagonal: keep j > k only
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (j0 + acc_row(r, g) <= k) aT[r] = 0.f;
      }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const frag<T> fa = chain<T>(aT, s2);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          mma(st[nt], TRV ? ld_free<T, true>(s_vut, LDK, 32 * nt, HD, 32 * jt + 16 * s2, c, g)
                          : ld_chain<T>(s_vut, LDV, 32 * nt + c, 32 * jt + 16 * s2, g), fa);
      }
    }
  }
  if (a.U.ptr != nullptr && k < L) {
    TI* dst = head_ptr_mut<TI>(a.U, b, h) + (int64_t)k * a.U.sl;
    const float su_mul = a.ws.hdr->su_mul;   // the state was built from vu * vu_scale
    bool half_format = false;
    if constexpr (sizeof(TI) == 2) half_format = a.u_half != 0;
    const float mul = half_format ? su_mul * kUHalfScale : su_mul;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) st[nt][r] *= mul;
    if (half_format) {   // half-precision cache format: fp16 bits of U * kUHalfScale, saturated
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) st[nt][r] = __builtin_amdgcn_fmed3f(st[nt][r], -kHalfMax, kHalfMax);
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = 32 * nt + 8 * q + 4 * g;
        if (n < HD) {
          if (half_format) st4<fp16_t>(reinterpret_cast<fp16_t*>(dst + n), pack4<fp16_t>(st[nt], q));
          else st4<TI>(dst + n, pack4<TI>(st[nt], q));
        }
      }
  }
}

// ---------------------------------------------------------------------------
template <typename T, typename TI, int HD>
__global__ __launch_bounds__(kThreads, sizeof(T) == 2 ? 2 : 1) void attn_kernel(FwdArgs a) {
  constexpr int KS = HD / 16;
  constexpr int HDP = HD < 32 ? 32 : HD;
  constexpr int NT = HDP / 32;
  constexpr int CK = attn_chunk<T, HD>();   // keys per chunk
  constexpr int KT = CK / 32;
  constexpr int QB = 128;
  constexpr int NBLK_Q = QB / kNB;   // snapshot blocks per workgroup
  constexpr int LDK = lds_ld_tr<T>(HD), LDV = lds_ld_chain<T>(kNB), LDA = lds_ld<T>(QB);
  constexpr bool PF = use_prefetch<T, HD>();
  constexpr bool TRV = sizeof(T) == 2;
  T* s_kc = reinterpret_cast<T*>(castle_smem);   // [CK][LDK]
  T* s_qu = s_kc + CK * LDK;                     // [CK][LDK]
  T* s_ub0 = s_qu + CK * LDK;                    // [NBLK_Q][CK][LDK]
  T* s_vct = s_ub0 + NBLK_Q * CK * LDK;          // fp32: [HDP][LDV] (transposed); 16-bit: [CK][LDK]
  T* s_a = s_vct + (TRV ? CK * LDK : vtile_elems<T, HD>());   // [CK][LDA]
  constexpr bool TL = attn_t_in_lds<T, HD>();
  constexpr int LDT = lds_ld<T>(kNB);
  T* s_t = s_a + CK * LDA;                                    // [QB][LDT], only if TL

  prio_by_band(blockIdx.x, a.s.cus);
  int rank, bh;
  work_item(a.s.B * a.s.H, rank, bh);
  const int qb = a.s.Lp / 128 - 1 - rank;   // the last query block sees the most keys
  const int b = bh / a.s.H, h = bh % a.s.H;
  const int lane = lane_id(), wave = wave_id(), c = lane & 31, g = lane >> 5;
  const int L = a.s.L;
  const float c1 = a.s.scale * kLog2e;
  const float su_mul = a.ws.hdr->su_mul;   // Su = su_mul * (the product built from vu * vu_scale)
  const bool unit_su = __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, su_mul)) == 0x3f800000;
  const int i0w = qb * QB + 32 * wave;
  const int i = i0w + c;
  const int Ifirst = (qb * QB) / kNB;
  const int Iw = i0w / kNB;
  const int jw = 32 * wave;                     // this wave's columns inside the A tile
  const int cb = (jw / kNB) * kNB;              // first column of its block
  const int nintra = ((jw % kNB) + 32) / 16;    // contraction steps of the in-block term

  const T* qc = prep_ptr<T>(a.ws.qc_p, bh, a.s.Lp, HD);   // pre-scaled by c1
  const T* kc = prep_ptr<T>(a.ws.kc_p, bh, a.s.Lp, HD);
  const T* vc = prep_ptr<T>(a.ws.vc_p, bh, a.s.Lp, HD);
  const T* qu = prep_ptr<T>(a.ws.qu_p, bh, a.s.Lp, HD);
  const T* ku = prep_ptr<T>(a.ws.ku_p, bh, a.s.Lp, HD);
  const T* tb = reinterpret_cast<const T*>(a.ws.t_blk) + (int64_t)bh * a.s.Lp * kNB;
  const T* snap = reinterpret_cast<const T*>(a.ws.usnap) + (int64_t)bh * snap_rows(a.s.nblk) * HD;

  frag<T> fqc[KS], fku[KS], ft[kNB / 16];   // c1 Qc rows, -c1 Ku rows, T' rows of this wave
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    fqc[s] = ldg_nat<T>(qc, HD, i, 16 * s + 8 * g, true);
    fku[s] = ldg_nat_scaled<T, T>(ku, HD, i, 16 * s + 8 * g, true, -c1);
  }
#pragma unroll
  for (int s = 0; s < kNB / 16; ++s) {
    ft[s] = ldg_nat<T>(tb, kNB, i, 16 * s + 8 * g, s < nintra);
    if (TL) *reinterpret_cast<frag<T>*>(s_t + (32 * wave + c) * LDT + 16 * s + 8 * g) = ft[s];
  }

  acc_t o[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) zero(o[nt]);
  float m = -INFINITY, l = 0.f;
  if (!TRV && HDP > HD) lds_zero(s_vct + HD * LDV, (HDP - HD) * LDV);

  int nchunks = (qb * QB + QB) / CK;
  if (nchunks > a.s.nblk * (kNB / CK)) nchunks = a.s.nblk * (kNB / CK);

  RowStage<T, T, CK, HD> pkc, pqu, pvr;
  ColStage<T, T, CK, HD> pvc;
  SnapStage<T, CK, HD> pub[NBLK_Q];
  auto load_chunk = [&](int ck) __attribute__((always_inline)) {   // chunk ck = keys [ck*CK, ck*CK + CK)
    const int Kb = ck * CK / kNB;
    pkc.load_flat(kc + (int64_t)ck * CK * HD);
    if (TRV) pvr.load_flat(vc + (int64_t)ck * CK * HD);
    else pvc.load(vc, HD, (int64_t)ck * CK, kNoRowLimit);
    pqu.load_flat(qu + (int64_t)ck * CK * HD);
#pragma unroll
    for (int q = 0; q < NBLK_Q; ++q) {
      const int blk = Ifirst + q;
      if (Kb < blk && blk < a.s.nblk) pub[q].load(snap + (usnap_off(blk) + (int64_t)ck * CK) * HD);
    }
  };
  auto store_chunk = [&](int ck) __attribute__((always_inline)) {
    const int Kb = ck * CK / kNB;
    pkc.store(s_kc, LDK);
    if (TRV) pvr.store(s_vct, LDK);
    else pvc.store(s_vct, LDV);
    pqu.store(s_qu, LDK);
#pragma unroll
    for (int q = 0; q < NBLK_Q; ++q) {
      const int blk = Ifirst + q;
      if (Kb < blk && blk < a.s.nblk) pub[q].store(s_ub0 + q * CK * LDK, LDK);
    }
  };

  // the row fragments are consumed before the loop as far as the wait counters are concerned:
  // otherwise every use inside the loop waits for the chunk prefetch issued after them
#pragma unroll
  for (int s = 0; s < KS; ++s) { asm volatile("" : "+v"(fqc[s])); asm volatile("" : "+v"(fku[s])); }
#pragma unroll
  for (int s = 0; s < kNB / 16; ++s)
    if (!TL) asm volatile("" : "+v"(ft[s]));
  if (PF) load_chunk(0);
  for (int ck = 0; ck < nchunks; ++ck) {
    const int Kb = ck * CK / kNB;
    __syncthreads();
    if (!PF) load_chunk(ck);
    store_chunk(ck);
    if (PF && ck + 1 < nchunks) load_chunk(ck + 1);   // in flight while this chunk is processed
    __syncthreads();
    const bool active = Kb <= Iw;
    if (active) {
      // gate tile for this wave's 32 source rows: A^T[j rows, k lanes]
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        acc_t aT;
        zero(aT);
#pragma unroll
        for (int s = 0; s < KS; ++s) mma(aT, fku[s], ld_nat<T>(s_qu, LDK, 32 * kt + c, 16 * s + 8 * g));
#pragma unroll
        for (int r = 0; r < 16; ++r) aT[r] = fast_rcp(1.f + fast_exp2(aT[r]));
        if (Kb == Iw) {
          const int kk = ck * CK + 32 * kt + c;
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (i0w + acc_row(r, g) <= kk) aT[r] = 0.f;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) st4<T>(s_a + (32 * kt + c) * LDA + jw + 8 * q + 4 * g, pack4<T>(aT, q));
      }
    }
    __syncthreads();
    if (active) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        const int k0 = ck * CK + 32 * kt;
        if (k0 > i0w + 31) continue;
        acc_t sc, su;
        zero(sc);
        zero(su);
#pragma unroll
        for (int s = 0; s < KS; ++s) mma(sc, ld_nat<T>(s_kc, LDK, 32 * kt + c, 16 * s + 8 * g), fqc[s]);
        // the in-block term first: its first two steps run for every wave, so the product that
        // starts the accumulator is unconditional and takes the zero as a constant operand
#pragma unroll
        for (int s = 0; s < kNB / 16; ++s)
          if (s < 2 || s < nintra)
            mma(su, ld_nat<T>(s_a, LDA, 32 * kt + c, cb + 16 * s + 8 * g), TL ? ld_nat<T>(s_t, LDT, 32 * wave + c, 16 * s + 8 * g) : ft[s]);
        if (Kb < Iw) {
          const T* ub = s_ub0 + (Iw - Ifirst) * CK * LDK;
#pragma unroll
          for (int s = 0; s < KS; ++s) mma(su, ld_nat<T>(ub, LDK, 32 * kt + c, 16 * s + 8 * g), fqc[s]);
        }

        // scores in log2 units: x = Sc' - Su' * sigmoid(Su)
        float mx = -INFINITY;
        if (unit_su) {   // the usual case (no range scaling of vu): one multiply per score less
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float sg = fast_rcp(1.f + fast_exp2(-su[r]));
            sc[r] = __builtin_fmaf(-su[r], sg, sc[r]);
          }
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float sut = su[r] * su_mul;
            const float sg = fast_rcp(1.f + fast_exp2(-sut));
            sc[r] = __builtin_fmaf(-sut, sg, sc[r]);
          }
        }
        if (k0 + 31 > i0w) {   // tile touches the diagonal: causal mask
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (k0 + acc_row(r, g) > i) sc[r] = -INFINITY;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sc[r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        if (__builtin_amdgcn_ballot_w64(mx > m) != 0) {   // some row maximum moved: rescale
          const float m_new = fmaxf(m, mx);
          const float alpha = fast_exp2(m - m_new);
          l *= alpha;
          m = m_new;
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[nt][r] *= alpha;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          sc[r] = fast_exp2(sc[r] - m);
          l += sc[r];
        }
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const frag<T> fp = chain<T>(sc, s2);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            mma(o[nt], TRV ? ld_free<T, true>(s_vct, LDK, 32 * nt, HD, 32 * kt + 16 * s2, c, g)
                           : ld_chain<T>(s_vct, LDV, 32 * nt + c, 32 * kt + 16 * s2, g), fp);
        }
      }
    }
  }
  const float lt = l + __shfl_xor(l, 32);
  if (i < L) {
    const float inv = 1.f / lt;
    TI* dst = head_ptr_mut<TI>(a.out, b, h) + (int64_t)i * a.out.sl;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) o[nt][r] *= inv;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = 32 * nt + 8 * q + 4 * g;
        if (n < HD) st4<TI>(dst + n, pack4<TI>(o[nt], q));
      }
    }
    if (g == 0) a.ws.lse[(int64_t)bh * a.s.Lp + i] = (m + __builtin_log2f(lt)) * kLn2;
  }
}

// ---------------------------------------------------------------------------
template <typename T, typename TI, int HD> static int launch_fwd_t(const FwdArgs& a, hipStream_t stream) {
  const int BH = a.s.B * a.s.H;
  constexpr int scan_lds = scan_lds_bytes<T, HD>(), attn_lds = attn_lds_bytes<T, HD>();
  if (attn_lds > kMaxLds) return -2;   // this (dtype, head dim) pair does not fit the 160 KB LDS
  static PerDeviceOnce once;
  bool& configured = once.flag();
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&scan_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, scan_lds) != hipSuccess) return -3;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, attn_lds) != hipSuccess) return -3;
    configured = true;
  }
  {
    ProfScope ps(kSlotPrep, stream);
    constexpr int PIECES_PER_ROW = HD / elem_traits<T>::vec16;
    if constexpr (sizeof(T) == 2)
      hipLaunchKernelGGL((amax_kernel<TI, HD>), dim3(kAmaxBlocks), dim3(kAmaxThreads), 0, stream, a.vu, a.s.H, a.s.L,
                         (int64_t)BH * a.s.L, a.ws.amax_part, &a.ws.hdr->status);
    hipLaunchKernelGGL((prep_kernel<T, TI, HD>), dim3((a.s.Lp * PIECES_PER_ROW + kThreads - 1) / kThreads, BH, 6), dim3(kThreads), 0, stream, a);
  }
  {
    ProfScope ps(kSlotScan, stream);
    hipLaunchKernelGGL((scan_kernel<T, TI, HD>), dim3(a.s.Lp / 128 * BH + (a.with_t ? a.s.nblk * BH : 0)), dim3(kThreads), scan_lds, stream, a);
  }
  {
    ProfScope ps(kSlotAttn, stream);
    hipLaunchKernelGGL((attn_kernel<T, TI, HD>), dim3(a.s.Lp / 128 * BH), dim3(kThreads), attn_lds, stream, a);
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <typename T, typename TI> static int launch_fwd_d(const FwdArgs& a, hipStream_t stream) {
  switch (a.s.d) {
    case 16: return launch_fwd_t<T, TI, 16>(a, stream);
    case 32: return launch_fwd_t<T, TI, 32>(a, stream);
    case 64: return launch_fwd_t<T, TI, 64>(a, stream);
    case 128: return launch_fwd_t<T, TI, 128>(a, stream);
    default: return -2;
  }
}

// The scan alone (snapshots of the lookahead state into a.ws.usnap from the operand copies the
// forward pass left): what the backward pass runs first when the forward snapshots were not kept.
template <typename T, typename TI, int HD> static int launch_scan_t(const FwdArgs& a, hipStream_t stream) {
  constexpr int scan_lds = scan_lds_bytes<T, HD>();
  static PerDeviceOnce once;
  bool& configured = once.flag();
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&scan_kernel<T, TI, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, scan_lds) != hipSuccess) return -3;
    configured = true;
  }
  ProfScope ps(kSlotScan, stream);
  hipLaunchKernelGGL((scan_kernel<T, TI, HD>), dim3(a.s.Lp / 128 * a.s.B * a.s.H + (a.with_t ? a.s.nblk * a.s.B * a.s.H : 0)), dim3(kThreads), scan_lds, stream, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
template <typename T, typename TI> static int launch_scan_d(const FwdArgs& a, hipStream_t stream) {
  switch (a.s.d) {
    case 16: return launch_scan_t<T, TI, 16>(a, stream);
    case 32: return launch_scan_t<T, TI, 32>(a, stream);
    case 64: return launch_scan_t<T, TI, 64>(a, stream);
    case 128: return launch_scan_t<T, TI, 128>(a, stream);
    default: return -2;
  }
}
int launch_scan(const FwdArgs& a, int dtype, bool bf16_operands, hipStream_t stream) {
  switch (dtype) {
    case 0: return launch_scan_d<float, float>(a, stream);
    case 1: return bf16_operands ? launch_scan_d<bf16_t, bf16_t>(a, stream) : launch_scan_d<fp16_t, bf16_t>(a, stream);
    case 2: return launch_scan_d<fp16_t, fp16_t>(a, stream);
    default: return -1;
  }
}

// bf16 tensors: operands are converted to fp16 on load (exact inside the fp16 range) and every
// operand produced inside the kernels is fp16, unless bf16_operands asks for bf16 MFMA operands.
int launch_fwd(const FwdArgs& a, int dtype, bool bf16_operands, hipStream_t stream) {
  switch (dtype) {
    case 0: return launch_fwd_d<float, float>(a, stream);
    case 1: return bf16_operands ? launch_fwd_d<bf16_t, bf16_t>(a, stream) : launch_fwd_d<fp16_t, bf16_t>(a, stream);
    case 2: return launch_fwd_d<fp16_t, fp16_t>(a, stream);
    default: return -1;
  }
}

}  // namespace castle
