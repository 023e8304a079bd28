// extern "C" surface of libcastle_hip.so (declared in include/castle_hip.h): argument
// validation, workspace carving and dispatch to the kernel launchers.  No torch types.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/castle_hip.h"
#include <stdlib.h>
#include "castle_params.h"
#include "castle_profile.h"
#include "castle_tiles.h"

namespace castle {
int launch_fwd(const FwdArgs& a, int dtype, bool bf16_operands, hipStream_t stream);
int launch_scan(const FwdArgs& a, int dtype, bool bf16_operands, hipStream_t stream);
int launch_bwd(const BwdArgs& a, int dtype, bool bf16_operands, hipStream_t stream);
int launch_decode(const DecodeArgs& a, int dtype, hipStream_t stream);
int launch_decode_flush(const DecodeArgs& a, int dtype, hipStream_t stream);
int launch_rope(const View4& src, const View4& dst, int B, int H, int L, int d, int dtype, int pos0, hipStream_t stream);
int decode_pick_splits(int BH, int t);
int decode_static_scratch(float** ptr);
int launch_small_linear(const void* x, const void* w, void* y, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldy,
                        int dtype, const void* norm_w, float eps, int act, const void* res, int64_t ldr, hipStream_t stream);
}  // namespace castle

namespace {

// compute units of the current device, looked up once per device
int device_cus() {
  static int cus[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
    cus[dev] = n;
  }
  return cus[dev];
}

using castle::kNB;

int elem_size(int dtype) {
  switch (dtype) {
    case CASTLE_F32: return 4;
    case CASTLE_BF16:
    case CASTLE_F16: return 2;
    default: return 0;
  }
}

bool head_dim_ok(int d) { return d == 16 || d == 32 || d == 64 || d == 128; }

int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

// upper limit of the dS / dSu tile buffers (they grow with B*H*L^2); beyond it the backward
// falls back to recomputing the score chain in its second kernel
constexpr int64_t kMaxScoreTileBytes = (int64_t)40 << 30;
// CASTLE_MAX_SCORE_TILE_BYTES in the environment overrides the limit (0 = never use the tiles)
// (read once, when the library first needs it, so that castle_bwd_workspace_bytes and castle_bwd
// cannot disagree)
int64_t max_score_tile_bytes() {
  static const int64_t limit = [] {
    const char* e = getenv("CASTLE_MAX_SCORE_TILE_BYTES");
    return e != nullptr ? strtoll(e, nullptr, 10) : kMaxScoreTileBytes;
  }();
  return limit;
}

struct Geometry {
  int Lp, nblk;
  int64_t lse_bytes, tblk_bytes, snap_bytes, mat_bytes, op_bytes;
  int64_t off_lse, off_t, off_tt, off_ttx, off_ops, total;
  int64_t bwd_total;
};
constexpr int64_t kHeaderBytes = 256 + 4 * castle::kAmaxBlocks;   // header + partial maxima, forward and backward alike

Geometry geometry(int B, int H, int L, int d, int es, int flags = 0) {
  Geometry g;
  g.Lp = (int)align_up(L, 128);
  g.nblk = g.Lp / kNB;
  const int64_t BH = (int64_t)B * H;
  g.lse_bytes = align_up(BH * g.Lp * 4, 256);
  g.tblk_bytes = align_up(BH * g.Lp * kNB * es, 256);
  g.snap_bytes = align_up(BH * castle::snap_rows(g.nblk) * d * es, 256);
  // dS / dSu tiles between the two backward kernels: the 16-bit paths use them
  g.mat_bytes = es == 2 ? align_up(BH * g.Lp * g.Lp * es, 256) : 0;
  // too long, or the caller asks for it: the query kernel recomputes the scores instead
  if (2 * g.mat_bytes > max_score_tile_bytes() || (flags & CASTLE_FLAG_RECOMPUTE_SCORES)) g.mat_bytes = 0;
  g.off_lse = kHeaderBytes;
  g.off_t = g.off_lse + g.lse_bytes;
  g.off_tt = g.off_t + g.tblk_bytes;
  g.off_ttx = g.off_tt + g.tblk_bytes;
  g.op_bytes = align_up(BH * g.Lp * d * es, 256);   // one operand in the compute type, padded to Lp rows
  g.off_ops = g.off_ttx + g.tblk_bytes;
  g.total = g.off_ops + 6 * g.op_bytes;            // the snapshots live in their own buffer (g.snap_bytes)
  // header, reverse-state snapshots, delta, dO copy, dS / dSu tiles, and the forward snapshots when they are recomputed
  g.bwd_total = kHeaderBytes + g.snap_bytes + g.lse_bytes + g.op_bytes + 2 * g.mat_bytes +
                ((flags & CASTLE_FLAG_RECOMPUTE_STATE) ? g.snap_bytes : 0);
  return g;
}

// pointer and strides must allow 16-byte vector access along d
bool view_ok(const castle_view4* v, int es, bool need_l) {
  if (v == nullptr || v->ptr == nullptr) return false;
  const int64_t q = 16 / es;
  if (reinterpret_cast<uintptr_t>(v->ptr) % 16 != 0) return false;
  if (v->stride_b % q != 0 || v->stride_h % q != 0) return false;
  if (need_l && v->stride_l % q != 0) return false;
  return true;
}

castle::View4 to_view(const castle_view4* v) {
  castle::View4 r;
  if (v == nullptr) {
    r.ptr = nullptr; r.sb = r.sh = r.sl = 0;
  } else {
    r.ptr = v->ptr; r.sb = v->stride_b; r.sh = v->stride_h; r.sl = v->stride_l;
  }
  return r;
}

int check_core(int B, int H, int L, int d, int dtype) {
  if (elem_size(dtype) == 0) return CASTLE_ERR_DTYPE;
  if (B <= 0 || H <= 0 || L <= 0 || !head_dim_ok(d)) return CASTLE_ERR_SHAPE;
  if ((int64_t)B * H > 65535) return CASTLE_ERR_SHAPE;   // grid.y of the small kernels
  if ((int64_t)B * H * ((L + 127) / 128) > 2147483647LL) return CASTLE_ERR_SHAPE;   // 1-D grid
  if (dtype == CASTLE_F32 && d > 64) return CASTLE_ERR_SHAPE;
  return CASTLE_OK;
}

castle::FwdWorkspace carve(void* base, void* state, const Geometry& g) {
  char* p = static_cast<char*>(base);
  castle::FwdWorkspace w;
  w.hdr = reinterpret_cast<castle::WsHeader*>(p);
  w.amax_part = reinterpret_cast<float*>(p + 256);
  w.lse = reinterpret_cast<float*>(p + g.off_lse);
  w.t_blk = p + g.off_t;
  w.tt_blk = p + g.off_tt;
  w.ttx_blk = p + g.off_ttx;
  w.usnap = state;
  w.qc_p = p + g.off_ops;
  w.kc_p = p + g.off_ops + g.op_bytes;
  w.vc_p = p + g.off_ops + 2 * g.op_bytes;
  w.qu_p = p + g.off_ops + 3 * g.op_bytes;
  w.ku_p = p + g.off_ops + 4 * g.op_bytes;
  w.vu_p = p + g.off_ops + 5 * g.op_bytes;
  return w;
}

}  // namespace

extern "C" {

int castle_abi_version(void) { return CASTLE_ABI_VERSION; }

const char* castle_error_string(int code) {
  switch (code) {
    case CASTLE_OK: return "ok";
    case CASTLE_ERR_DTYPE: return "unknown element type";
    case CASTLE_ERR_SHAPE: return "unsupported shape (head dim must be 16/32/64/128, fp32 needs d <= 64, B*H <= 65535)";
    case CASTLE_ERR_LAUNCH: return "HIP launch or configuration error";
    case CASTLE_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case CASTLE_ERR_ARG: return "NULL or misaligned tensor view";
    case CASTLE_ERR_SCRATCH: return "problem too large for the static scratch of the entry point that allocates nothing";
    default: return "unknown error";
  }
}

int64_t castle_fwd_workspace_bytes(int B, int H, int L, int d, int dtype) {
  const int rc = check_core(B, H, L, d, dtype);
  if (rc != CASTLE_OK) return rc;
  return geometry(B, H, L, d, elem_size(dtype)).total;
}

int64_t castle_fwd_state_bytes(int B, int H, int L, int d, int dtype) {
  const int rc = check_core(B, H, L, d, dtype);
  if (rc != CASTLE_OK) return rc;
  const int64_t n = geometry(B, H, L, d, elem_size(dtype)).snap_bytes;
  return n > 0 ? n : 256;   // a single block has no snapshots; keep the buffer non-empty
}

int castle_fwd(const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
               const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
               int B, int H, int L, int d, int dtype, float scale, int flags,
               const castle_view4* out, const castle_view4* U,
               void* workspace, int64_t workspace_bytes, void* state, int64_t state_bytes, void* stream) {
  int rc = check_core(B, H, L, d, dtype);
  if (rc != CASTLE_OK) return rc;
  const int es = elem_size(dtype);
  const castle_view4* in[] = {qc, kc, vc, qu, ku, vu, out};
  for (const castle_view4* v : in)
    if (!view_ok(v, es, true)) return CASTLE_ERR_ARG;
  const bool want_U = U != nullptr && U->ptr != nullptr;
  if (want_U && !view_ok(U, es, true)) return CASTLE_ERR_ARG;
  if ((flags & CASTLE_FLAG_U_HALF) && dtype != CASTLE_BF16) return CASTLE_ERR_DTYPE;   // the format replaces bf16 only
  const Geometry g = geometry(B, H, L, d, es);
  if (workspace == nullptr || reinterpret_cast<uintptr_t>(workspace) % 256 != 0 || workspace_bytes < g.total)
    return CASTLE_ERR_WORKSPACE;
  if (state == nullptr || reinterpret_cast<uintptr_t>(state) % 256 != 0 || state_bytes < g.snap_bytes)
    return CASTLE_ERR_WORKSPACE;

  castle::FwdArgs a;
  a.s.B = B; a.s.H = H; a.s.L = L; a.s.d = d; a.s.Lp = g.Lp; a.s.nblk = g.nblk; a.s.scale = scale;
  a.s.rotary = (flags & CASTLE_FLAG_ROTARY) != 0;
  a.s.cus = device_cus();
  a.qc = to_view(qc); a.kc = to_view(kc); a.vc = to_view(vc);
  a.qu = to_view(qu); a.ku = to_view(ku); a.vu = to_view(vu);
  a.out = to_view(out);
  a.U = to_view(want_U ? U : nullptr);
  a.u_half = (flags & CASTLE_FLAG_U_HALF) != 0;
  a.ws = carve(workspace, state, g);
  return castle::launch_fwd(a, dtype, (flags & CASTLE_FLAG_BF16_OPERANDS) != 0, static_cast<hipStream_t>(stream));
}

int64_t castle_bwd_workspace_bytes(int B, int H, int L, int d, int dtype, int flags) {
  const int rc = check_core(B, H, L, d, dtype);
  if (rc != CASTLE_OK) return rc;
  const Geometry g = geometry(B, H, L, d, elem_size(dtype), flags);
  return g.bwd_total;
}

int castle_bwd(const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
               const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
               const castle_view4* out, const castle_view4* dout,
               int B, int H, int L, int d, int dtype, float scale, int flags,
               const castle_view4* dqc, const castle_view4* dkc, const castle_view4* dvc,
               const castle_view4* dqu, const castle_view4* dku, const castle_view4* dvu,
               const void* fwd_workspace, int64_t fwd_workspace_bytes,
               const void* fwd_state, int64_t fwd_state_bytes,
               void* bwd_workspace, int64_t bwd_workspace_bytes, void* stream) {
  int rc = check_core(B, H, L, d, dtype);
  if (rc != CASTLE_OK) return rc;
  const int es = elem_size(dtype);
  const castle_view4* in[] = {qc, kc, vc, qu, ku, vu, out, dout, dqc, dkc, dvc, dqu, dku, dvu};
  for (const castle_view4* v : in)
    if (!view_ok(v, es, true)) return CASTLE_ERR_ARG;
  const Geometry g = geometry(B, H, L, d, es, flags);
  if (fwd_workspace == nullptr || reinterpret_cast<uintptr_t>(fwd_workspace) % 256 != 0 || fwd_workspace_bytes < g.total)
    return CASTLE_ERR_WORKSPACE;
  if (bwd_workspace == nullptr || reinterpret_cast<uintptr_t>(bwd_workspace) % 256 != 0 ||
      bwd_workspace_bytes < g.bwd_total)
    return CASTLE_ERR_WORKSPACE;
  const bool recompute_state = (flags & CASTLE_FLAG_RECOMPUTE_STATE) != 0;
  if (!recompute_state &&
      (fwd_state == nullptr || reinterpret_cast<uintptr_t>(fwd_state) % 256 != 0 || fwd_state_bytes < g.snap_bytes))
    return CASTLE_ERR_WORKSPACE;

  castle::BwdArgs a;
  a.s.B = B; a.s.H = H; a.s.L = L; a.s.d = d; a.s.Lp = g.Lp; a.s.nblk = g.nblk; a.s.scale = scale;
  a.s.rotary = (flags & CASTLE_FLAG_ROTARY) != 0;
  a.s.cus = device_cus();
  a.qc = to_view(qc); a.kc = to_view(kc); a.vc = to_view(vc);
  a.qu = to_view(qu); a.ku = to_view(ku); a.vu = to_view(vu);
  a.out = to_view(out); a.dout = to_view(dout);
  a.dqc = to_view(dqc); a.dkc = to_view(dkc); a.dvc = to_view(dvc);
  a.dqu = to_view(dqu); a.dku = to_view(dku); a.dvu = to_view(dvu);
  char* bw = static_cast<char*>(bwd_workspace);
  // forward snapshots: the caller's, or recomputed into the tail of this call's own workspace
  void* state = recompute_state ? bw + (g.bwd_total - g.snap_bytes) : const_cast<void*>(fwd_state);
  a.ws = carve(const_cast<void*>(fwd_workspace), state, g);
  a.bhdr = reinterpret_cast<castle::BwdHeader*>(bw);
  a.amax_part = reinterpret_cast<float*>(bw + 256);
  bw += kHeaderBytes;
  a.gsnap = bw;
  a.delta = reinterpret_cast<float*>(bw + g.snap_bytes);
  a.dout_p = bw + g.snap_bytes + g.lse_bytes;
  a.ds_mat = g.mat_bytes ? bw + g.snap_bytes + g.lse_bytes + g.op_bytes : nullptr;
  a.dsu_mat = g.mat_bytes ? bw + g.snap_bytes + g.lse_bytes + g.op_bytes + g.mat_bytes : nullptr;
  if (recompute_state) {   // the scan again, from the operand copies the forward pass left
    castle::FwdArgs f;
    f.s = a.s;
    f.qc = a.qc; f.kc = a.kc; f.vc = a.vc; f.qu = a.qu; f.ku = a.ku; f.vu = a.vu;
    f.out = a.out;
    f.U = to_view(nullptr);
    f.ws = a.ws;
    f.with_t = 0;
    rc = castle::launch_scan(f, dtype, (flags & CASTLE_FLAG_BF16_OPERANDS) != 0, static_cast<hipStream_t>(stream));
    if (rc != 0) return rc;
  }
  return castle::launch_bwd(a, dtype, (flags & CASTLE_FLAG_BF16_OPERANDS) != 0, static_cast<hipStream_t>(stream));
}

int64_t castle_decode_workspace_bytes(int B, int H, int d, int t_max) {
  if (B <= 0 || H <= 0 || !head_dim_ok(d) || t_max < 0) return CASTLE_ERR_SHAPE;
  return align_up((int64_t)B * H * 64 * (d + 2) * 4, 256);
}

static int decode_step_common(const castle_view4* U, const castle_view4* qu_cache,
                              const castle_view4* kc_cache, const castle_view4* vc_cache,
                              int t, const int* t_device, int capacity,
                              const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
                              const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
                              int B, int H, int d, int dtype, float scale, int flags,
                              const castle_view4* out, const castle_deferred* deferred,
                              void* workspace, int64_t workspace_bytes, bool static_scratch, void* stream) {
  const int es = elem_size(dtype);
  if (es == 0) return CASTLE_ERR_DTYPE;
  if ((flags & CASTLE_FLAG_U_HALF) && dtype != CASTLE_BF16) return CASTLE_ERR_DTYPE;
  if (B <= 0 || H <= 0 || t < 0 || capacity <= 0 || !head_dim_ok(d) || (int64_t)B * H > 65535) return CASTLE_ERR_SHAPE;
  if (t_device == nullptr && t >= capacity) return CASTLE_ERR_SHAPE;   // row t would be written past the buffers
  const castle_view4* caches[] = {U, qu_cache, kc_cache, vc_cache};
  for (const castle_view4* v : caches)
    if (!view_ok(v, es, true)) return CASTLE_ERR_ARG;
  const castle_view4* tok[] = {qc, kc, vc, qu, ku, vu, out};
  for (const castle_view4* v : tok)
    if (!view_ok(v, es, false)) return CASTLE_ERR_ARG;
  if (deferred != nullptr) {
    if (!view_ok(&deferred->vu_ring, es, true) || !view_ok(&deferred->gates, 4, false)) return CASTLE_ERR_ARG;
    if (deferred->base < 0 || (deferred->base_device != nullptr && reinterpret_cast<uintptr_t>(deferred->base_device) % 4 != 0))
      return CASTLE_ERR_ARG;
    // host-side counts: the pending sources must all fit the ring
    if (t_device == nullptr && deferred->base_device == nullptr && deferred->base > t) return CASTLE_ERR_SHAPE;
  }
  // with a device-side count the split must not depend on it: sized for a full cache
  const int splits = castle::decode_pick_splits(B * H, t_device != nullptr ? capacity : t);
  if (static_scratch) {
    // the per-GPU array replaces the caller's workspace; nothing is allocated on this path
    if ((int64_t)B * H * splits * (d + 2) * 4 > castle::kDecodeStaticScratchBytes) return CASTLE_ERR_SCRATCH;
    float* p = nullptr;
    if (castle::decode_static_scratch(&p) != 0) return CASTLE_ERR_LAUNCH;
    workspace = p;
  } else if (workspace == nullptr || reinterpret_cast<uintptr_t>(workspace) % 256 != 0 ||
             workspace_bytes < castle_decode_workspace_bytes(B, H, d, t)) {
    return CASTLE_ERR_WORKSPACE;
  }

  castle::DecodeArgs a;
  a.B = B; a.H = H; a.d = d; a.t = t; a.scale = scale;
  a.t_dev = t_device; a.capacity = capacity;
  a.rotary = (flags & CASTLE_FLAG_ROTARY) != 0;
  a.u_half = (flags & CASTLE_FLAG_U_HALF) != 0;
  a.splits = splits;
  a.U = to_view(U); a.qu_cache = to_view(qu_cache); a.kc_cache = to_view(kc_cache); a.vc_cache = to_view(vc_cache);
  a.qc = to_view(qc); a.kc = to_view(kc); a.vc = to_view(vc);
  a.qu = to_view(qu); a.ku = to_view(ku); a.vu = to_view(vu);
  a.out = to_view(out);
  a.part = static_cast<float*>(workspace);
  a.pend_vu = to_view(deferred != nullptr ? &deferred->vu_ring : nullptr);
  a.pend_gate = to_view(deferred != nullptr ? &deferred->gates : nullptr);
  a.base0 = deferred != nullptr ? deferred->base : 0;
  a.base0_dev = deferred != nullptr ? deferred->base_device : nullptr;
  return castle::launch_decode(a, dtype, static_cast<hipStream_t>(stream));
}

int castle_decode_step(const castle_view4* U, const castle_view4* qu_cache,
                       const castle_view4* kc_cache, const castle_view4* vc_cache, int t, int capacity,
                       const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
                       const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
                       int B, int H, int d, int dtype, float scale, int flags,
                       const castle_view4* out, const castle_deferred* deferred,
                       void* workspace, int64_t workspace_bytes, void* stream) {
  return decode_step_common(U, qu_cache, kc_cache, vc_cache, t, nullptr, capacity, qc, kc, vc, qu, ku, vu,
                            B, H, d, dtype, scale, flags, out, deferred, workspace, workspace_bytes, false, stream);
}

int castle_decode_step_static(const castle_view4* U, const castle_view4* qu_cache,
                              const castle_view4* kc_cache, const castle_view4* vc_cache,
                              int t, const int32_t* t_device, int capacity,
                              const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
                              const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
                              int B, int H, int d, int dtype, float scale, int flags,
                              const castle_view4* out, const castle_deferred* deferred, void* stream) {
  if (t_device != nullptr && reinterpret_cast<uintptr_t>(t_device) % 4 != 0) return CASTLE_ERR_ARG;
  return decode_step_common(U, qu_cache, kc_cache, vc_cache, t_device != nullptr ? 0 : t, t_device, capacity,
                            qc, kc, vc, qu, ku, vu, B, H, d, dtype, scale, flags, out, deferred, nullptr, 0, true, stream);
}

int castle_decode_step_device_count(const castle_view4* U, const castle_view4* qu_cache,
                                    const castle_view4* kc_cache, const castle_view4* vc_cache,
                                    const int32_t* t_device, int capacity,
                                    const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
                                    const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
                                    int B, int H, int d, int dtype, float scale, int flags,
                                    const castle_view4* out, const castle_deferred* deferred,
                                    void* workspace, int64_t workspace_bytes, void* stream) {
  if (t_device == nullptr || reinterpret_cast<uintptr_t>(t_device) % 4 != 0) return CASTLE_ERR_ARG;
  return decode_step_common(U, qu_cache, kc_cache, vc_cache, 0, t_device, capacity, qc, kc, vc, qu, ku, vu,
                            B, H, d, dtype, scale, flags, out, deferred, workspace, workspace_bytes, false, stream);
}

int castle_decode_flush(const castle_view4* U, const castle_view4* qu_cache, int t, const castle_deferred* deferred,
                        int B, int H, int d, int dtype, float scale, int flags, void* stream) {
  const int es = elem_size(dtype);
  if (es == 0) return CASTLE_ERR_DTYPE;
  if ((flags & CASTLE_FLAG_U_HALF) && dtype != CASTLE_BF16) return CASTLE_ERR_DTYPE;
  if (B <= 0 || H <= 0 || t < 0 || !head_dim_ok(d) || (int64_t)B * H > 65535) return CASTLE_ERR_SHAPE;
  if (!view_ok(U, es, true) || !view_ok(qu_cache, es, true) || deferred == nullptr) return CASTLE_ERR_ARG;
  if (!view_ok(&deferred->vu_ring, es, true) || !view_ok(&deferred->gates, 4, false)) return CASTLE_ERR_ARG;
  if (deferred->base < 0 || deferred->base > t) return CASTLE_ERR_SHAPE;
  if (t == 0 || castle::decode_base(deferred->base, t) == t) return CASTLE_OK;   // nothing pending
  castle::DecodeArgs a = {};
  a.B = B; a.H = H; a.d = d; a.t = t; a.scale = scale;
  a.U = to_view(U); a.qu_cache = to_view(qu_cache);
  a.pend_vu = to_view(&deferred->vu_ring); a.pend_gate = to_view(&deferred->gates);
  a.base0 = deferred->base;
  a.u_half = (flags & CASTLE_FLAG_U_HALF) != 0;
  return castle::launch_decode_flush(a, dtype, static_cast<hipStream_t>(stream));
}

int castle_rope(const castle_view4* x, const castle_view4* out, int B, int H, int L, int d, int dtype,
                int first_position, void* stream) {
  const int es = elem_size(dtype);
  if (es == 0) return CASTLE_ERR_DTYPE;
  if (B <= 0 || H <= 0 || L <= 0 || first_position < 0 || !head_dim_ok(d) || (int64_t)B * H > 65535) return CASTLE_ERR_SHAPE;
  if (!view_ok(x, es, true) || !view_ok(out, es, true)) return CASTLE_ERR_ARG;
  return castle::launch_rope(to_view(x), to_view(out), B, H, L, d, dtype, first_position, static_cast<hipStream_t>(stream));
}

int castle_small_linear_fused(const void* x, const void* w, void* y, int M, int N, int K,
                              int64_t ldx, int64_t ldw, int64_t ldy, int dtype,
                              const void* norm_weight, float eps, int activation,
                              const void* residual, int64_t ldr, void* stream) {
  if (dtype != CASTLE_BF16 && dtype != CASTLE_F16) return CASTLE_ERR_DTYPE;
  if (M <= 0 || N <= 0 || K <= 0 || K % 8 != 0 || N % 2 != 0) return CASTLE_ERR_SHAPE;
  if (x == nullptr || w == nullptr || y == nullptr) return CASTLE_ERR_ARG;
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(w) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(y) % 4 != 0 || ldx % 8 != 0 || ldw % 8 != 0 || ldy % 2 != 0)
    return CASTLE_ERR_ARG;
  if (activation != CASTLE_ACT_NONE && activation != CASTLE_ACT_GELU) return CASTLE_ERR_ARG;
  if (norm_weight != nullptr && (reinterpret_cast<uintptr_t>(norm_weight) % 16 != 0 || !(eps >= 0.f))) return CASTLE_ERR_ARG;
  if (residual != nullptr && (reinterpret_cast<uintptr_t>(residual) % 4 != 0 || ldr % 2 != 0)) return CASTLE_ERR_ARG;
  return castle::launch_small_linear(x, w, y, M, N, K, ldx, ldw, ldy, dtype, norm_weight, eps, activation, residual, ldr,
                                     static_cast<hipStream_t>(stream));
}

int castle_small_linear(const void* x, const void* w, void* y, int M, int N, int K,
                        int64_t ldx, int64_t ldw, int64_t ldy, int dtype, void* stream) {
  return castle_small_linear_fused(x, w, y, M, N, K, ldx, ldw, ldy, dtype, nullptr, 0.f, CASTLE_ACT_NONE, nullptr, 0, stream);
}

int castle_profile_enable(int on) { return castle::profile_enable(on); }

int castle_profile_read(int* slots, float* ms, int max_records) {
  if (slots == nullptr || ms == nullptr || max_records < 0) return CASTLE_ERR_ARG;
  return castle::profile_read(slots, ms, max_records);
}

}  // extern "C"
