// Device-side tile toolkit for the CASTLE kernels (gfx950 / CDNA4, wave64).
//
// Every contraction in the kernels is a 32x32 MFMA tile:
//   bf16 : v_mfma_f32_32x32x16_bf16   (one instruction per 16-deep step)
//   fp16 : v_mfma_f32_32x32x16_f16
//   fp32 : 8 x v_mfma_f32_32x32x2_f32 (same register fragments, 8 elements deep per lane)
// Lane l = (c, g) with c = l % 32, g = l / 32.
//   operand fragment : 8 elements of the contraction axis for free index c.
//                      "natural" order : slot e <-> contraction index 16*s + 8*g + e
//                      "chained" order : slot e <-> contraction index 16*s + 8*(e/4) + 4*g + e%4
//   accumulator tile : 16 floats; register r <-> row 8*(r/4) + 4*g + r%4, column c.
// An accumulator tile whose ROW index is the next contraction index converts in
// registers into two operand fragments in chained order (registers 0-7 and 8-15);
// the partner operand is then read from LDS with ld_chain().
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "castle_params.h"

namespace castle {

// "Done once per device" flag for host-side kernel configuration (the dynamic-LDS limit of a
// kernel is a per-device attribute).  Racing callers at worst configure twice, which is harmless.
struct PerDeviceOnce {
  bool done[64] = {};
  bool& flag() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    return done[dev];
  }
};

typedef __bf16 bf16_t;
typedef _Float16 fp16_t;
template <typename T, int N> using vec = T __attribute__((ext_vector_type(N)));
typedef vec<float, 16> acc_t;
template <typename T> using frag = vec<T, 8>;
// memory views of the vectors: never assume more than 16-byte (or natural, if smaller) alignment
template <typename T> using frag_mem = vec<T, 8> __attribute__((aligned(16)));
template <typename T> using vec4_mem = vec<T, 4> __attribute__((aligned(8)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr int64_t kNoRowLimit = (int64_t)1 << 40;   // row_end of staging loads from padded arrays
constexpr int kNB = 64;        // block size of the state snapshots (rows per block)
constexpr int kThreads = 256;  // 4 waves per workgroup in every tiled kernel
constexpr int kMaxLds = 160 * 1024;

template <typename T> struct elem_traits;
template <> struct elem_traits<bf16_t> { static constexpr int vec16 = 8; };
template <> struct elem_traits<fp16_t> { static constexpr int vec16 = 8; };
template <> struct elem_traits<float> { static constexpr int vec16 = 4; };

// padded leading dimension of an LDS tile with `cols` payload columns (16 bytes of pad)
template <typename T> __host__ __device__ constexpr int lds_ld(int cols) { return cols + elem_traits<T>::vec16; }
// The same for a 16-bit tile that is also read with transpose reads (ds_read_b64_tr_b16): on rows 132 or 136
// elements apart such a read takes 48 cycles instead of 26 (measured; 40 ... 152 otherwise all take 26, and
// 16-byte reads are slow only at 48, 80 and 144), so a 128-column tile gets rows of 152.
template <typename T> __host__ __device__ constexpr int lds_ld_tr(int cols) {
  return sizeof(T) == 2 && cols == 128 ? 152 : lds_ld<T>(cols);
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
// The wave index is read through readfirstlane so that the compiler knows it is uniform:
// every branch that depends on it then becomes a scalar branch.  This matters for
// correctness, not only speed: MFMA instructions do not honour the EXEC mask, so an MFMA
// inside a branch the compiler believes to be per-lane can execute for a wave that should
// have skipped it.  No MFMA in these kernels may sit under a condition that is not derived
// from wave_id(), blockIdx or kernel arguments.
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }
__device__ __forceinline__ int acc_row(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

__device__ __forceinline__ void mma(acc_t& c, const frag<bf16_t>& a, const frag<bf16_t>& b) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ void mma(acc_t& c, const frag<fp16_t>& a, const frag<fp16_t>& b) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ void mma(acc_t& c, const frag<float>& a, const frag<float>& b) {
#pragma unroll
  for (int t = 0; t < 8; ++t) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], c, 0, 0, 0);
}

__device__ __forceinline__ void zero(acc_t& c) {
#pragma unroll
  for (int r = 0; r < 16; ++r) c[r] = 0.f;
}

template <typename T> __device__ __forceinline__ frag<T> zero_frag() {
  frag<T> f;
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (T)0.f;
  return f;
}

// registers 8*s .. 8*s+7 of an accumulator tile as an operand fragment (chained order)
template <typename T> __device__ __forceinline__ frag<T> chain(const acc_t& c, int s) {
  vec<float, 8> v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = c[8 * s + e];
  return __builtin_convertvector(v, frag<T>);
}

// store 4 packed elements (8 bytes for 16-bit types, 16 for fp32)
template <typename T> __device__ __forceinline__ void st4(T* p, vec<T, 4> v) { *reinterpret_cast<vec4_mem<T>*>(p) = v; }
// the same for data that is written once and read once by a later kernel: kept out of the way of what the caches hold
template <typename T> __device__ __forceinline__ void st4_stream(T* p, vec<T, 4> v) { __builtin_nontemporal_store(v, reinterpret_cast<vec4_mem<T>*>(p)); }

// 8 contiguous elements tile[row][col .. col+7]
template <typename T> __device__ __forceinline__ frag<T> ld_nat(const T* tile, int ld, int row, int col) {
  return *reinterpret_cast<const frag_mem<T>*>(tile + row * ld + col);
}
// chained order: tile[row][col0+4g .. +3] and tile[row][col0+8+4g .. +3]   (col0 multiple of 16)
template <typename T> __device__ __forceinline__ frag<T> ld_chain(const T* tile, int ld, int row, int col0, int g) {
  const T* p = tile + row * ld + col0 + 4 * g;
  vec<T, 4> lo = *reinterpret_cast<const vec4_mem<T>*>(p);
  vec<T, 4> hi = *reinterpret_cast<const vec4_mem<T>*>(p + 8);
  frag<T> f;
#pragma unroll
  for (int e = 0; e < 4; ++e) { f[e] = lo[e]; f[4 + e] = hi[e]; }
  return f;
}

// element-wise conversion between the I/O type TI and the compute type T (same width);
// bf16 -> fp16 goes through fp32 and is exact for values inside the fp16 range
template <typename T, typename TI, int N> __device__ __forceinline__ vec<T, N> cvt_vec(vec<TI, N> x) {
  if constexpr (__is_same(T, TI)) {
    return x;
  } else {
    static_assert(sizeof(T) == sizeof(TI), "I/O and compute types must have the same width");
    return __builtin_convertvector(__builtin_convertvector(x, vec<float, N>), vec<T, N>);
  }
}

// ---- transposed operand fragments straight from a row-major LDS tile ---------------------
// ds_read_b64_tr_b16: inside each group of 16 lanes, lane i slot e receives element (i % 4) of
// the 4-element row whose address lane (4e + i/4) supplied.  If lanes 4e..4e+3 of a group point
// at columns n .. n+15 of contraction row rho(e), lane i ends up with rows rho(0..3) of its own
// column n + i.  Two such reads build an operand fragment whose FREE index (n0 + c) sits on
// lanes from data stored [contraction][free], in natural or chained contraction order.
typedef short v4i16_t __attribute__((ext_vector_type(4)));
template <typename T> __device__ __forceinline__ vec<T, 4> lds_tr4(const T* p) {
  static_assert(sizeof(T) == 2, "transpose reads exist for 16-bit elements");
  typedef v4i16_t __attribute__((address_space(3))) * lds_ptr;
  return __builtin_bit_cast(vec<T, 4>, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p));
}
// rm: row-major tile [contraction][free], ld multiple of 4.  Returns the fragment for free
// index n0 + c (n0 multiple of 32) and the 16 contraction rows starting at contr0.
// 16-bit types use transpose reads; fp32 gathers.  Lanes whose free index is >= free_limit
// (only possible when the tile has fewer than 32 payload columns) get zeros.
template <typename T, bool CHAINED>
__device__ __forceinline__ frag<T> ld_free(const T* rm, int ld, int n0, int free_limit, int contr0, int c, int g) {
  frag<T> f;
  if constexpr (sizeof(T) == 2) {
    const int lp = c & 15;
    const T* p = rm + (contr0 + (CHAINED ? 4 : 8) * g + (lp >> 2)) * ld + n0 + 16 * (c >> 4) + 4 * (lp & 3);
    const vec<T, 4> lo = lds_tr4<T>(p);
    const vec<T, 4> hi = lds_tr4<T>(p + (CHAINED ? 8 : 4) * ld);
#pragma unroll
    for (int e = 0; e < 4; ++e) { f[e] = lo[e]; f[4 + e] = hi[e]; }
    if (free_limit < n0 + 32 && n0 + c >= free_limit) f = zero_frag<T>();
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = contr0 + (CHAINED ? 8 * (e >> 2) + 4 * g + (e & 3) : 8 * g + e);
      f[e] = n0 + c < free_limit ? rm[j * ld + n0 + c] : (T)0.f;
    }
  }
  return f;
}

// natural fragment straight from global memory (row-major, unit inner stride); zeros when !ok
template <typename T, typename TI = T>
__device__ __forceinline__ frag<T> ldg_nat(const TI* base, int64_t row_stride, int64_t row, int col, bool ok) {
  if (!ok) return zero_frag<T>();
  return cvt_vec<T, TI, 8>(*reinterpret_cast<const frag_mem<TI>*>(base + row * row_stride + col));
}

// ---- global -> LDS staging -------------------------------------------------
// Copies a ROWS x COLS tile whose first row is global row `row0`; rows >= `row_end` are
// zero-filled.  dst is row-major with leading dimension lds_ld<T>(COLS).
template <typename T, int ROWS, int COLS, typename TI = T>
__device__ __forceinline__ void stage_rows(T* dst, const TI* src, int64_t row_stride, int64_t row0, int64_t row_end) {
  constexpr int V = elem_traits<T>::vec16;
  constexpr int VPR = COLS / V;
  constexpr int LD = lds_ld<T>(COLS);
  typedef vec<T, V> v16;
  typedef vec<TI, V> v16i;
  for (int v = threadIdx.x; v < ROWS * VPR; v += kThreads) {
    int r = v / VPR, cv = v % VPR;
    v16 x;
#pragma unroll
    for (int e = 0; e < V; ++e) x[e] = (T)0.f;
    if (row0 + r < row_end) x = cvt_vec<T, TI, V>(*reinterpret_cast<const v16i*>(src + (row0 + r) * row_stride + cv * V));
    *reinterpret_cast<v16*>(dst + r * LD + cv * V) = x;
  }
}

// Transposed copy: dst[c][r] = src[row0 + r][c]; dst has COLS payload rows (callers that
// need more rows zero them once) and leading dimension lds_ld<T>(ROWS).
template <typename T, int ROWS, int COLS, typename TI = T>
__device__ __forceinline__ void stage_rows_t(T* dst, const TI* src, int64_t row_stride, int64_t row0, int64_t row_end) {
  constexpr int V = elem_traits<T>::vec16;
  constexpr int VPR = COLS / V;
  constexpr int LD = lds_ld<T>(ROWS);
  typedef vec<T, V> v16;
  typedef vec<TI, V> v16i;
  typedef vec<T, 4> v4;
  for (int p = threadIdx.x; p < (ROWS / 4) * VPR; p += kThreads) {
    int rg = p / VPR, cv = p % VPR;
    v16 x[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int e = 0; e < V; ++e) x[q][e] = (T)0.f;
      int64_t row = row0 + 4 * rg + q;
      if (row < row_end) x[q] = cvt_vec<T, TI, V>(*reinterpret_cast<const v16i*>(src + row * row_stride + cv * V));
    }
#pragma unroll
    for (int e = 0; e < V; ++e) {
      v4 y;
#pragma unroll
      for (int q = 0; q < 4; ++q) y[q] = x[q][e];
      *reinterpret_cast<vec4_mem<T>*>(dst + (cv * V + e) * LD + 4 * rg) = y;
    }
  }
}

// zero `count` elements of LDS (count multiple of 8)
template <typename T> __device__ __forceinline__ void lds_zero(T* dst, int count) {
  for (int i = threadIdx.x * 8; i < count; i += kThreads * 8) *reinterpret_cast<frag_mem<T>*>(dst + i) = zero_frag<T>();
}


// 4 consecutive rows (registers 4q..4q+3) of an accumulator tile as a packed vector of T
template <typename T> __device__ __forceinline__ vec<T, 4> pack4(const acc_t& c, int q) {
  vec<float, 4> v = {c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]};
  return __builtin_convertvector(v, vec<T, 4>);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
// sigmoid(y) given z = y * log2(e)
__device__ __forceinline__ float sigmoid_l2(float z) { return fast_rcp(1.f + fast_exp2(-z)); }

// natural fragment from global memory multiplied by `mul` in fp32 before the conversion to T
template <typename T, typename TI = T>
__device__ __forceinline__ frag<T> ldg_nat_scaled(const TI* base, int64_t row_stride, int64_t row, int col, bool ok, float mul) {
  if (!ok) return zero_frag<T>();
  vec<float, 8> v = __builtin_convertvector(*reinterpret_cast<const frag_mem<TI>*>(base + row * row_stride + col), vec<float, 8>);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] *= mul;
  return __builtin_convertvector(v, frag<T>);
}

// leading dimension of a tile that is read with ld_chain (8-byte halves): 8 bytes of pad for
// 16-bit types make both the transposed stores and the chained reads bank-conflict free
template <typename T> __host__ __device__ constexpr int lds_ld_chain(int cols) { return cols + 4; }

// Two-phase staging of a ROWS x COLS tile: load() brings the 16-byte pieces of this thread into
// registers (zeros beyond row_end), store() converts them to T and writes the row-major LDS tile.
// Splitting the phases lets a kernel issue the loads of the next tile before computing on the
// current one.
template <typename T, typename TI, int ROWS, int COLS, int THREADS = kThreads>
struct RowStage {
  static constexpr int V = elem_traits<T>::vec16;
  static constexpr int VPR = COLS / V;
  static constexpr int TOTAL = ROWS * VPR;
  static constexpr int N = (TOTAL + THREADS - 1) / THREADS;
  vec<TI, V> r[N];

  __device__ __forceinline__ void load(const TI* src, int64_t row_stride, int64_t row0, int64_t row_end, int tid = threadIdx.x) {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int v = tid + n * THREADS;
#pragma unroll
      for (int e = 0; e < V; ++e) r[n][e] = (TI)0.f;
      if (v < TOTAL && row0 + v / VPR < row_end)
        r[n] = *reinterpret_cast<const vec<TI, V>*>(src + (row0 + v / VPR) * row_stride + (v % VPR) * V);
    }
  }
  // Same for a tile whose ROWS rows of COLS elements are contiguous in memory and all exist (the
  // operand copies in the compute type): piece v of the tile sits at tile + v * V.
  __device__ __forceinline__ void load_flat(const TI* tile, int tid = threadIdx.x) {
    static_assert(TOTAL % THREADS == 0 || TOTAL < THREADS, "tile must split evenly over the threads");
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int v = tid + n * THREADS;
      if (TOTAL >= THREADS || v < TOTAL) r[n] = *reinterpret_cast<const vec<TI, V>*>(tile + v * V);
    }
  }
  __device__ __forceinline__ void store(T* dst, int ld, int tid = threadIdx.x) const {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int v = tid + n * THREADS;
      if (v < TOTAL) *reinterpret_cast<vec<T, V>*>(dst + (v / VPR) * ld + (v % VPR) * V) = cvt_vec<T, TI, V>(r[n]);
    }
  }
  // for tiles whose rows are only 8-byte aligned (leading dimension from lds_ld_chain)
  __device__ __forceinline__ void store_halves(T* dst, int ld, int tid = threadIdx.x) const {
    constexpr int HV = V / 2;
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int v = tid + n * THREADS;
      if (v < TOTAL) {
        const vec<T, V> x = cvt_vec<T, TI, V>(r[n]);
        typedef vec<T, HV> __attribute__((aligned(8))) half_mem;
        vec<T, HV> lo, hi;
#pragma unroll
        for (int e = 0; e < HV; ++e) { lo[e] = x[e]; hi[e] = x[HV + e]; }
        T* q = dst + (v / VPR) * ld + (v % VPR) * V;
        *reinterpret_cast<half_mem*>(q) = lo;
        *reinterpret_cast<half_mem*>(q + HV) = hi;
      }
    }
  }
  __device__ __forceinline__ void store_scaled(T* dst, int ld, float mul, int tid = threadIdx.x) const {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int v = tid + n * THREADS;
      if (v < TOTAL) {
        vec<float, V> f = __builtin_convertvector(r[n], vec<float, V>);
#pragma unroll
        for (int e = 0; e < V; ++e) f[e] *= mul;
        *reinterpret_cast<vec<T, V>*>(dst + (v / VPR) * ld + (v % VPR) * V) = __builtin_convertvector(f, vec<T, V>);
      }
    }
  }
};

// Same for the transposed copy dst[c][r] = src[row0 + r][c].  A thread owns 4 rows x V columns.
// Lane -> patch map: within 16 consecutive lanes the patches cover 2 column groups x 8 row
// groups, which makes the 8-byte LDS stores hit 16 distinct bank pairs while every load
// instruction of a wave still reads 8 complete rows.
template <typename T, typename TI, int ROWS, int COLS>
struct ColStage {
  static constexpr int V = elem_traits<T>::vec16;
  static constexpr int VPR = COLS / V;
  static constexpr int RG = ROWS / 4;
  static constexpr int TOTAL = RG * VPR;
  static constexpr int N = (TOTAL + kThreads - 1) / kThreads;
  static_assert(VPR % 2 == 0 && RG % 8 == 0, "tile shape not supported by the patch map");
  vec<TI, V> r[N][4];

  static __device__ __forceinline__ void patch(int p, int& rg, int& cv) {
    const int rest = p >> 4;
    cv = (rest % (VPR / 2)) * 2 + (p & 1);
    rg = (rest / (VPR / 2)) * 8 + ((p >> 1) & 7);
  }
  __device__ __forceinline__ void load(const TI* src, int64_t row_stride, int64_t row0, int64_t row_end) {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int p = threadIdx.x + n * kThreads;
      int rg, cv;
      patch(p, rg, cv);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int e = 0; e < V; ++e) r[n][q][e] = (TI)0.f;
        const int64_t row = row0 + 4 * rg + q;
        if (p < TOTAL && row < row_end) r[n][q] = *reinterpret_cast<const vec<TI, V>*>(src + row * row_stride + cv * V);
      }
    }
  }
  __device__ __forceinline__ void store(T* dst, int ld, float mul = 1.f) const {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int p = threadIdx.x + n * kThreads;
      if (p >= TOTAL) continue;
      int rg, cv;
      patch(p, rg, cv);
      vec<float, V> f[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) f[q] = __builtin_convertvector(r[n][q], vec<float, V>);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        vec<float, 4> y = {f[0][e] * mul, f[1][e] * mul, f[2][e] * mul, f[3][e] * mul};
        st4<T>(dst + (cv * V + e) * ld + 4 * rg, __builtin_convertvector(y, vec<T, 4>));
      }
    }
  }
};

// Patch staging: a group of GROUP threads stages one ROWS x COLS tile; a thread owns 4-row x
// 16-byte patches, loaded once from global memory, from which it can write the row-major LDS
// tile, the transposed LDS tile, or both.  load() only issues the global loads, so several
// tiles (one PatchStage each, handled by different waves) are in flight together and the
// loads of the next tile can be issued before the current one is consumed.  `lt` is the index
// of the thread inside its group (0 .. GROUP-1).
template <typename T, typename TI, int ROWS, int COLS, int GROUP>
struct PatchStage {
  static constexpr int V = elem_traits<T>::vec16;
  static constexpr int VPR = COLS / V;
  static constexpr int RG = ROWS / 4;
  static constexpr int TOTAL = RG * VPR;
  static constexpr int N = (TOTAL + GROUP - 1) / GROUP;
  static_assert(VPR % 2 == 0 && RG % 8 == 0, "tile shape not supported by the patch map");
  vec<TI, V> r[N][4];

  static __device__ __forceinline__ void patch(int p, int& rg, int& cv) {
    const int rest = p >> 4;
    cv = (rest % (VPR / 2)) * 2 + (p & 1);
    rg = (rest / (VPR / 2)) * 8 + ((p >> 1) & 7);
  }
  __device__ __forceinline__ void load(int lt, const TI* src, int64_t row_stride, int64_t row0, int64_t row_end) {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int p = lt + n * GROUP;
      int rg, cv;
      patch(p, rg, cv);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int e = 0; e < V; ++e) r[n][q][e] = (TI)0.f;
        const int64_t row = row0 + 4 * rg + q;
        if (p < TOTAL && row < row_end) r[n][q] = *reinterpret_cast<const vec<TI, V>*>(src + row * row_stride + cv * V);
      }
    }
  }
  // row-major tile dst[r][c]; HALVES = true writes 8-byte halves (rows only 8-byte aligned)
  template <bool HALVES = false>
  __device__ __forceinline__ void store_rows(int lt, T* dst, int ld, float mul = 1.f) const {
    constexpr int HV = V / 2;
    typedef vec<T, HV> __attribute__((aligned(8))) half_mem;
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int p = lt + n * GROUP;
      if (p >= TOTAL) continue;
      int rg, cv;
      patch(p, rg, cv);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        vec<float, V> f = __builtin_convertvector(r[n][q], vec<float, V>);
#pragma unroll
        for (int e = 0; e < V; ++e) f[e] *= mul;
        const vec<T, V> x = __builtin_convertvector(f, vec<T, V>);
        T* w = dst + (4 * rg + q) * ld + cv * V;
        if constexpr (HALVES) {
          vec<T, HV> lo, hi;
#pragma unroll
          for (int e = 0; e < HV; ++e) { lo[e] = x[e]; hi[e] = x[HV + e]; }
          *reinterpret_cast<half_mem*>(w) = lo;
          *reinterpret_cast<half_mem*>(w + HV) = hi;
        } else {
          *reinterpret_cast<vec<T, V>*>(w) = x;
        }
      }
    }
  }
  // transposed tile dst[c][r]
  __device__ __forceinline__ void store_cols(int lt, T* dst, int ld, float mul = 1.f) const {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int p = lt + n * GROUP;
      if (p >= TOTAL) continue;
      int rg, cv;
      patch(p, rg, cv);
      vec<float, V> f[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) f[q] = __builtin_convertvector(r[n][q], vec<float, V>);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        vec<float, 4> y = {f[0][e] * mul, f[1][e] * mul, f[2][e] * mul, f[3][e] * mul};
        st4<T>(dst + (cv * V + e) * ld + 4 * rg, __builtin_convertvector(y, vec<T, 4>));
      }
    }
  }
};

// Work-item order of the row-block kernels.  The grid is 1-D with nrow * BH workgroups; item
// `id` maps to row block `rank = id / BH` of head `bh = id % BH`.  Callers order `rank` from the
// longest row block to the shortest, so across ALL heads the expensive blocks are dispatched
// first (the causal triangle otherwise leaves a long tail), and because workgroups are dealt
// round-robin to the 8 XCDs, head bh always lands on XCD (bh % 8) whenever BH is a multiple of
// 8: the K/V/state rows of one head stay in one L2.
__device__ __forceinline__ void work_item(int BH, int& rank, int& bh) {
  rank = blockIdx.x / BH;
  bh = blockIdx.x % BH;
}

// ---- state snapshots -------------------------------------------------------------------
// A snapshot holds one state row (HD values) per key.  Keys are grouped by 32 ("snapshot
// tile", 32*HD elements, tiles in key order); inside a tile the 16-byte pieces (V values of one
// key) are stored piece-column major: element (key c, column n) sits at
//   (n / V) * 32 * V + c * V + n % V.
// The producers hold the state transposed in MFMA accumulators (rows n, one key per lane), so
// each of their store instructions covers 512 contiguous bytes; consumers read whole tiles as
// one contiguous run of pieces.
template <typename T> __device__ __forceinline__ int snap_elem(int c, int n) {
  constexpr int V = elem_traits<T>::vec16;
  return (n / V) * 32 * V + c * V + n % V;
}

// Stores acc tiles st[nt] (rows n = 32 nt + .., lane (c, g) = key c of the tile) into one snapshot tile.
template <typename T, int HD, int NT>
__device__ __forceinline__ void store_snap_tile(T* tile, const acc_t (&st)[NT], int c, int g) {
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = 32 * nt + 8 * q + 4 * g;
      if (n < HD) st4_stream<T>(tile + snap_elem<T>(c, n), pack4<T>(st[nt], q));
    }
}

// The natural-order operand fragment (columns 16 s + 8 g .. + 7 of key c) straight from a snapshot tile.
template <typename T> __device__ __forceinline__ frag<T> ldg_snap_nat(const T* tile, int c, int col) {
  constexpr int V = elem_traits<T>::vec16;
  if constexpr (V == 8) {
    return __builtin_nontemporal_load(reinterpret_cast<const frag_mem<T>*>(tile + snap_elem<T>(c, col)));   // read once
  } else {
    frag<T> f;
    const vec<T, 4> lo = *reinterpret_cast<const vec<T, 4>*>(tile + snap_elem<T>(c, col));
    const vec<T, 4> hi = *reinterpret_cast<const vec<T, 4>*>(tile + snap_elem<T>(c, col + 4));
#pragma unroll
    for (int e = 0; e < 4; ++e) { f[e] = lo[e]; f[4 + e] = hi[e]; }
    return f;
  }
}

// Two-phase staging of ROWS (a multiple of 32) snapshot rows into a row-major LDS tile.
template <typename T, int ROWS, int COLS>
struct SnapStage {
  static constexpr int V = elem_traits<T>::vec16;
  static constexpr int VPR = COLS / V;
  static constexpr int TOTAL = ROWS * VPR;
  static constexpr int N = (TOTAL + kThreads - 1) / kThreads;
  static_assert(ROWS % 32 == 0, "whole snapshot tiles only");
  vec<T, V> r[N];

  // src: first element of the first tile (the tiles of consecutive key groups are contiguous)
  __device__ __forceinline__ void load(const T* src, int tid = threadIdx.x) {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int v = tid + n * kThreads;
      if (v < TOTAL) r[n] = __builtin_nontemporal_load(reinterpret_cast<const vec<T, V>*>(src + (int64_t)v * V));   // read once
    }
  }
  __device__ __forceinline__ void store(T* dst, int ld, int tid = threadIdx.x) const {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int v = tid + n * kThreads;
      if (v < TOTAL) {
        const int tile = v / (32 * VPR), piece = (v / 32) % VPR, c = v % 32;
        *reinterpret_cast<vec<T, V>*>(dst + (32 * tile + c) * ld + piece * V) = r[n];
      }
    }
  }
};

// Rotary position embedding over the interleaved pairs (x[2i], x[2i+1]) of a row of HD elements:
// angle = pos * 10000^(-2i/HD) (lookahead_keys_attention.py:71-73,106-112 apply it to qc, kc, qu,
// ku, vu through a third-party module; this is the standard form).  `inverse` rotates by the
// opposite angle, which is the transpose: what the gradient of a rotated operand needs.
__device__ __forceinline__ vec<float, 2> rope_rot(float x0, float x1, float pos, int pair, int HD, bool inverse) {
  const float inv_freq = exp2f(-(float)(2 * pair) / (float)HD * 13.287712379549449f);   // 10000^(-2i/HD)
  // the hardware sine / cosine take their argument in turns; reduce it to [0, 1) first
  const float turns = pos * inv_freq * 0.15915494309189535f;
  const float fr = turns - floorf(turns);
  float sn = __builtin_amdgcn_sinf(fr);
  const float cs = __builtin_amdgcn_cosf(fr);
  if (inverse) sn = -sn;
  vec<float, 2> y = {x0 * cs - x1 * sn, x1 * cs + x0 * sn};
  return y;
}
// the same on two lvalues (vector elements cannot be bound to references)
#define CASTLE_ROPE_PAIR(X0, X1, POS, PAIR, HD_, INV)                          \
  do {                                                                         \
    const vec<float, 2> y_ = rope_rot((X0), (X1), (POS), (PAIR), (HD_), (INV)); \
    (X0) = y_[0];                                                              \
    (X1) = y_[1];                                                              \
  } while (0)

// ---- range control ------------------------------------------------------------------------
// Partial maxima of |x| over a (B, H, L, HD) view: kAmaxBlocks workgroups, one partial each.  The
// consumers reduce the partials themselves (amax_from_partials), so no atomics and no clearing.
constexpr int kAmaxThreads = 1024;
template <typename TI, int HD>
__global__ __launch_bounds__(kAmaxThreads) void amax_kernel(View4 x, int H, int L, int64_t rows, float* part, int* status) {
  constexpr int V = elem_traits<TI>::vec16;
  constexpr int VPR = HD / V;
  constexpr int UN = 4;   // independent loads in flight per thread
  if (status != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *status = 0;
  float m = 0.f;
  const int64_t pieces = rows * VPR;
  const int64_t stride = (int64_t)gridDim.x * kAmaxThreads;
  for (int64_t p0 = (int64_t)blockIdx.x * kAmaxThreads + threadIdx.x; p0 < pieces; p0 += UN * stride) {
    vec<TI, V> v[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int64_t p = p0 + u * stride;
#pragma unroll
      for (int e = 0; e < V; ++e) v[u][e] = (TI)0.f;
      if (p < pieces) {
        const int64_t row = p / VPR;
        const int cv = (int)(p % VPR);
        const int64_t bh = row / L, l = row % L;
        v[u] = *reinterpret_cast<const vec<TI, V>*>(reinterpret_cast<const TI*>(x.ptr) + (bh / H) * x.sb + (bh % H) * x.sh + l * x.sl + cv * V);
      }
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const vec<float, V> f = __builtin_convertvector(v[u], vec<float, V>);
#pragma unroll
      for (int e = 0; e < V; ++e) m = fmaxf(m, fabsf(f[e]));   // fmaxf drops NaNs
    }
  }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) m = fmaxf(m, __shfl_xor(m, o));
  __shared__ float s_m[kAmaxThreads / 64];
  if ((threadIdx.x & 63) == 0) s_m[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kAmaxThreads / 64; ++w) m = fmaxf(m, s_m[w]);
    part[blockIdx.x] = fminf(m, 3.0e38f);   // an infinite input counts as the largest finite value
  }
}
// max of the partials, by every thread of a wave (64 lanes x 4 partials)
__device__ __forceinline__ float amax_from_partials(const float* part) {
  static_assert(kAmaxBlocks == 256, "one load of four partials per lane");
  const vec<float, 4> v = *reinterpret_cast<const vec<float, 4>*>(part + 4 * lane_id());
  float m = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) m = fmaxf(m, __shfl_xor(m, o));
  return m;
}
// the power of two 2^k with  2^lo <= x * 2^k < 2^(lo+1)  (1 for x == 0)
__device__ __forceinline__ float pow2_placing(float x, int lo) {
  if (!(x > 0.f)) return 1.f;
  int e;
  (void)frexpf(x, &e);   // x = f * 2^e, f in [0.5, 1)
  int k = lo + 1 - e;
  k = k < -100 ? -100 : (k > 100 ? 100 : k);
  return ldexpf(1.f, k);
}
// vu_scale: the largest power of two <= 1 with  L * max|vu| * scale <= 2^15
__device__ __forceinline__ float vu_scale_for(float amax_vu, int L) {
  const float bound = amax_vu * (float)L;
  if (!(bound > 32768.f)) return 1.f;
  int e;
  (void)frexpf(bound, &e);   // bound < 2^e
  return ldexpf(1.f, 15 - e);
}
constexpr float kHalfMax = 65504.f;

// Issue priority of a workgroup from its place in the launch order.  Workgroups are handed out in
// index order, one per CU until every CU has one, then a second each, and so on; of two workgroups
// that share a CU the hardware favours the older, and the younger crawls (measured in the attention
// kernel: 3.8 against 5.5 us per chunk) and finishes late.  Raising the priority of every second
// band of `cus` workgroups turns that around for the pairs formed at the start (the shorter rows
// finish early and make room), leaves the long rows ahead of the late, short arrivals, and makes
// the two waves of a SIMD take strict turns instead of interleaving (both get faster).
__device__ __forceinline__ void prio_by_band(int id, int cus) {
  if (cus > 0 && ((id / cus) & 1)) __builtin_amdgcn_s_setprio(3);
}

// head bh of an operand copy in the compute type ([B*H][Lp][HD] contiguous, rows >= L zero)
template <typename T> __device__ __forceinline__ const T* prep_ptr(const void* base, int bh, int Lp, int HD) {
  return reinterpret_cast<const T*>(base) + (int64_t)bh * Lp * HD;
}

// offsets (in rows) of block I inside the snapshot arrays
__host__ __device__ inline int64_t usnap_off(int64_t I) { return (int64_t)kNB * I * (I - 1) / 2; }   // I >= 1, I*kNB rows
__host__ __device__ inline int64_t gsnap_off(int64_t I) { return (int64_t)kNB * I * (I + 1) / 2; }   // I <= nblk-2, (I+1)*kNB rows
__host__ __device__ inline int64_t snap_rows(int64_t nblk) { return (int64_t)kNB * nblk * (nblk - 1) / 2; }

}  // namespace castle
