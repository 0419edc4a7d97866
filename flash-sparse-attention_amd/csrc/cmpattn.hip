// Compressed attention (queries against the compressed keys / values), the
// block-importance scores derived from it and the top-k block selection, gfx950.
//
//   cmpattn_fwd   : query-major flash attention over tiles of 64 compressed keys
//                   staged in LDS; rows are (query, head-in-group) pairs so one
//                   K/V tile serves the whole GQA group; S^T = K Q^T with one row
//                   per lane, online softmax in registers, O^T += V^T P^T.
//   cmpattn_bwd   : delta, a query-major dQ kernel of the same shape, and the
//                   shared key-major dK/dV kernel (dkdv_kernel.h).
//   cmp_score     : probabilities of the first head of every group, fp32.
//   cmp_topk      : per query: weighted 5-tap re-binning into selection blocks,
//                   forced blocks, cast to bf16, top-k by (value desc, id asc),
//                   ascending ids, ids above the own block -> -1.
//
// Semantics: nsa_ref/ops/compressed_attention.py:27-156 (forward; key j visible
// to query i iff i >= j*stride + ks - 1, rows without a visible key give O = 0,
// LSE = -inf), :195-518 (backward), :832-930 (score), :1006-1158 (transform),
// :1272-1315 (selection).
#include "fsa_common.h"
#include "dkdv_kernel.h"

namespace fsa {

struct CmpParams {
  const void* q;
  const void* k;
  const void* v;
  const void* d_o;
  void* o;
  void* dq;
  float* lse;          // [Hq, N]
  const float* delta;  // [Hq, N]
  int64_t q_sn, q_sh, k_sn, k_sh, v_sn, v_sh, o_sn, o_sh, do_sn, do_sh;
  const int32_t* cu_q;
  const int32_t* cu_k;
  int64_t n_tokens;
  int g;
  int kernel_size, kernel_stride;
  int window;  // sliding-window mode: key p visible to query i iff i - window <= p <= i
  float scale, scale_log2;
  // score / top-k
  float* score;        // [Hkv, N, score_ld]
  int64_t score_ld;
  int score_head_step;  // q head that scores kv head h = h * score_head_step (g: first head of the group)
  int rebin;           // cmp_score writes block scores (taps 1 2 2 2 1 over groups of 4 keys) instead of probabilities
};

constexpr int CMP_MODE_COMPRESSED = 0;
constexpr int CMP_MODE_WINDOW = 1;   // the same query-major kernels over raw keys with a causal band mask
constexpr int CMP_BK = 64;      // compressed keys per tile
constexpr int CMP_ROWS = 128;   // rows per work-group (4 waves x 32)

template <int D> struct CmpLds {
  static constexpr int KS = D + 16;  // 32 B pad: the transposing reads of K^T (dQ kernel) run conflict-free, with 16 B they do not
  static constexpr int VS = D + 16;
  static constexpr int BYTES = (CMP_BK * KS + CMP_BK * VS) * 2;
};

// A K / V tile of CMP_BK rows travels as 16-byte chunks, chunk c = tid + 256 j of thread tid: row c / (D / 8),
// which is tid / (D / 8) + j * ROWS_PER_STEP.  The loads are buffer loads: step j has a scalar descriptor of its
// own (first row of the step, as many bytes as the step has rows left in the sequence) and every step uses the
// same 32-bit lane offset (kv_tile_offset), which never changes - no per-load vector arithmetic at all, and the
// rows past the end of the sequence (last tile only) come back as zeros from the descriptor's range check.
template <typename T, int D> struct KvTileRegs {
  static constexpr int CPR = D / 8;                  // 16-byte chunks per row
  static constexpr int ROWS_PER_STEP = 256 / CPR;
  static constexpr int N = CMP_BK / ROWS_PER_STEP;   // chunks per thread and tensor
  typename Elem<T>::vec8 k[N], v[N];
};
template <typename T, int D>
__device__ __forceinline__ uint32_t kv_tile_offset(int64_t sn, int tid) {
  constexpr int CPR = KvTileRegs<T, D>::CPR;
  return (uint32_t)((tid / CPR) * sn * (int64_t)sizeof(T)) + (tid % CPR) * 16;   // host: CMP_BK * sn * sizeof(T) < 2^32
}
template <typename T, int D, int N>
__device__ __forceinline__ void kv_rows_load(typename Elem<T>::vec8 (&r)[N], const T* base, int64_t sn, uint32_t off,
                                             int row0, int n_valid) {
  constexpr int RPS = KvTileRegs<T, D>::ROWS_PER_STEP;
  const int64_t row_bytes = sn * (int64_t)sizeof(T);
  const char* tile = reinterpret_cast<const char*>(base) + row0 * row_bytes;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const int rows = min(n_valid - j * RPS, RPS);  // rows of this step inside the sequence
    const uint32_t bytes = rows > 0 ? (uint32_t)((rows - 1) * row_bytes) + D * (uint32_t)sizeof(T) : 0u;
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(tile + j * RPS * row_bytes), 0, (int)bytes, 0x00020000);
    r[j] = __builtin_bit_cast(typename Elem<T>::vec8, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0));
  }
}
// kv_tile_load issues the global loads of a tile into registers, kv_tile_store parks them in LDS: in two steps,
// so that the rows of the next tile can travel while the current one is used.
template <typename T, int D, bool HAS_V = true>
__device__ __forceinline__ void kv_tile_load(KvTileRegs<T, D>& r, const T* kbase, int64_t k_sn, uint32_t k_off,
                                             const T* vbase, int64_t v_sn, uint32_t v_off, int row0, int n_valid,
                                             int tid) {
  kv_rows_load<T, D>(r.k, kbase, k_sn, k_off, row0, n_valid);
  if (HAS_V) kv_rows_load<T, D>(r.v, vbase, v_sn, v_off, row0, n_valid);
}
template <typename T, int D, bool HAS_V = true>
__device__ __forceinline__ void kv_tile_store(const KvTileRegs<T, D>& r, T* Ks, T* Vs, int tid) {
  constexpr int KS = CmpLds<D>::KS, VS = CmpLds<D>::VS;
  constexpr int CPR = KvTileRegs<T, D>::CPR, RPS = KvTileRegs<T, D>::ROWS_PER_STEP;
#pragma unroll
  for (int j = 0; j < KvTileRegs<T, D>::N; ++j) {
    const int row = tid / CPR + j * RPS, col = tid % CPR;
    store16(&Ks[row * KS + col * 8], r.k[j]);
    if (HAS_V) store16(&Vs[row * VS + col * 8], r.v[j]);
  }
}
template <typename T, int D, bool HAS_V = true>
__device__ __forceinline__ void stage_kv_tile(const T* kbase, int64_t k_sn, uint32_t k_off, const T* vbase, int64_t v_sn,
                                              uint32_t v_off, int row0, int n_valid, T* Ks, T* Vs, int tid) {
  KvTileRegs<T, D> r;
  kv_tile_load<T, D, HAS_V>(r, kbase, k_sn, k_off, vbase, v_sn, v_off, row0, n_valid, tid);
  kv_tile_store<T, D, HAS_V>(r, Ks, Vs, tid);
}

// Per-row and per-work-group visible key range [lo, hi] (inclusive) in both modes.
template <int MODE> struct KeyRange {
  static __device__ __forceinline__ int hi(const CmpParams& p, int qi, int nc) {
    if (MODE == CMP_MODE_WINDOW) return min(qi, nc - 1);
    const int j = qi >= p.kernel_size - 1 ? (qi - p.kernel_size + 1) / p.kernel_stride : -1;
    return min(j, nc - 1);
  }
  static __device__ __forceinline__ int lo(const CmpParams& p, int qi) {
    return MODE == CMP_MODE_WINDOW ? max(0, qi - p.window) : 0;
  }
};

// ---------------------------------------------------------------- forward ----
template <typename T, int D, int MODE>
__global__ void __launch_bounds__(256, (D <= 128 ? 2 : 1))
cmpattn_fwd_kernel(CmpParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef typename Elem<T>::vec4 vec4;
  constexpr int KS = CmpLds<D>::KS, VS = CmpLds<D>::VS;
  constexpr int NA = CMP_BK / 32, NKS = D / 16, NDT = D / 32, NJ = CMP_BK / 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Ks = reinterpret_cast<T*>(smem);
  T* Vs = Ks + CMP_BK * KS;

  const int s = blockIdx.y, h = blockIdx.z;
  const int q0 = p.cu_q[s], lq = p.cu_q[s + 1] - q0;
  const int k0 = MODE == CMP_MODE_WINDOW ? q0 : p.cu_k[s];
  const int nc = MODE == CMP_MODE_WINDOW ? lq : p.cu_k[s + 1] - k0;
  const int rows_total = lq * p.g;
  const int row_lo = blockIdx.x * CMP_ROWS;
  if (row_lo >= rows_total) return;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int r = row_lo + wv * 32 + col;
  const bool valid = r < rows_total;
  const int rr = valid ? r : rows_total - 1;
  const int qi = rr / p.g, head = rr - qi * p.g;
  const int hq_i = h * p.g + head;
  const T* qrow = reinterpret_cast<const T*>(p.q) + (int64_t)(q0 + qi) * p.q_sn + (int64_t)hq_i * p.q_sh + hh * (D / 2);
  vec8 qreg[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) qreg[ks] = load16<vec8>(qrow + ks * 8);
  // keys visible to this row and to the rows of the work-group
  const int jmax = KeyRange<MODE>::hi(p, qi, nc), jmin = KeyRange<MODE>::lo(p, qi);
  const int qi_first = row_lo / p.g, qi_last = (min(rows_total, row_lo + CMP_ROWS) - 1) / p.g;
  const int n_keys = KeyRange<MODE>::hi(p, qi_last, nc) + 1;                 // end of the work-group's key range
  const int jt0 = KeyRange<MODE>::lo(p, qi_first) / CMP_BK * CMP_BK;          // its tile-aligned start

  const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)h * p.k_sh;
  const T* vbase = reinterpret_cast<const T*>(p.v) + (int64_t)h * p.v_sh;
  const uint32_t k_off = kv_tile_offset<T, D>(p.k_sn, tid), v_off = kv_tile_offset<T, D>(p.v_sn, tid);
  const T* vtr = Vs + (4 * hh + ((lane & 15) >> 2)) * VS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  float m = -INFINITY, l = 0.f;  // m in raw (unscaled) score units
  f32x16 oacc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;

  constexpr bool PREFETCH = D <= 128;  // the next tile waits in registers where the budget allows
  KvTileRegs<T, D> nxt;
  if (PREFETCH && jt0 < n_keys) kv_tile_load<T, D>(nxt, kbase, p.k_sn, k_off, vbase, p.v_sn, v_off, k0 + jt0, nc - jt0, tid);
  for (int jt = jt0; jt < n_keys; jt += CMP_BK) {
    if (jt != jt0) __syncthreads();
    if (PREFETCH) {
      kv_tile_store<T, D>(nxt, Ks, Vs, tid);
      if (jt + CMP_BK < n_keys)
        kv_tile_load<T, D>(nxt, kbase, p.k_sn, k_off, vbase, p.v_sn, v_off, k0 + jt + CMP_BK, nc - jt - CMP_BK, tid);
    } else {
      stage_kv_tile<T, D>(kbase, p.k_sn, k_off, vbase, p.v_sn, v_off, k0 + jt, nc - jt, Ks, Vs, tid);
    }
    __syncthreads();
    f32x16 acc[NA];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
      for (int a = 0; a < NA; ++a) {  // consecutive products on different accumulators
        vec8 kf = load16<vec8>(&Ks[(a * 32 + col) * KS + hh * (D / 2) + ks * 8]);
        acc[a] = Elem<T>::mfma32(kf, qreg[ks], acc[a]);
      }
    const int limit = jmax - jt, limit_lo = jmin - jt;
    float mx = m;
    // tiles that every row of the wave sees completely need no mask
    if (!__all(limit >= CMP_BK - 1 && limit_lo <= 0)) {
#pragma unroll
      for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = a * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
          if (!(key <= limit && key >= limit_lo)) acc[a][i] = -INFINITY;
        }
    }
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, acc[a][i]);
    mx = fmaxf(mx, xor32(mx));
    // The reference maximum m moves only when some row of the wave outgrows it by more than 2^8: until then
    // the probabilities are taken relative to the older, smaller maximum (at most 256, exact in the final
    // quotient) and the accumulators need no rescaling.  (-inf) - (-inf) is NaN and compares false.
    if (__any((mx - m) * p.scale_log2 > 8.f)) {
      // m = -inf -> 0; a row that keeps its maximum -> 1; a row that has seen no key yet has nothing to rescale
      const float alpha = mx == -INFINITY ? 1.f : exp2f((m - mx) * p.scale_log2);
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
      m = mx;
    }
    const float mref = (m == -INFINITY) ? 0.f : m * p.scale_log2;
    float lsum = 0.f;
    vec8 pk[NJ];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pv = fast_exp2(acc[a][i] * p.scale_log2 - mref);
        lsum += pv;
        pk[a * 2 + (i >> 3)][i & 7] = (T)pv;
      }
    lsum += xor32(lsum);
    l += lsum;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        vec8 vf = lds_read_tr8<T>(vtr + 16 * j * VS + dt * 32, 8 * VS);
        oacc[dt] = Elem<T>::mfma32(vf, pk[j], oacc[dt]);
      }
    }
  }
  if (!valid) return;
  const float inv_l = l > 0.f ? 1.f / l : 0.f;
  T* orow = reinterpret_cast<T*>(p.o) + (int64_t)(q0 + qi) * p.o_sn + (int64_t)hq_i * p.o_sh + 4 * hh;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      vec4 x;
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = (T)(oacc[dt][4 * qd + e] * inv_l);
      store8(orow + dt * 32 + 8 * qd, x);
    }
  if (hh == 0) p.lse[(int64_t)hq_i * p.n_tokens + q0 + qi] = l > 0.f ? m * p.scale_log2 + log2f(l) : -INFINITY;
}

// --------------------------------------------------------------------- dq ----
template <typename T, int D, int MODE>
__global__ void __launch_bounds__(256, (D <= 128 ? 2 : 1))
cmpattn_bwd_dq_kernel(CmpParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef typename Elem<T>::vec4 vec4;
  constexpr int KS = CmpLds<D>::KS, VS = CmpLds<D>::VS;
  constexpr int NA = CMP_BK / 32, NKS = D / 16, NDT = D / 32, NJ = CMP_BK / 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Ks = reinterpret_cast<T*>(smem);
  T* Vs = Ks + CMP_BK * KS;

  const int s = blockIdx.y, h = blockIdx.z;
  const int q0 = p.cu_q[s], lq = p.cu_q[s + 1] - q0;
  const int k0 = MODE == CMP_MODE_WINDOW ? q0 : p.cu_k[s];
  const int nc = MODE == CMP_MODE_WINDOW ? lq : p.cu_k[s + 1] - k0;
  const int rows_total = lq * p.g;
  const int row_lo = blockIdx.x * CMP_ROWS;
  if (row_lo >= rows_total) return;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int r = row_lo + wv * 32 + col;
  const bool valid = r < rows_total;
  const int rr = valid ? r : rows_total - 1;
  const int qi = rr / p.g, head = rr - qi * p.g;
  const int hq_i = h * p.g + head;
  const T* qrow = reinterpret_cast<const T*>(p.q) + (int64_t)(q0 + qi) * p.q_sn + (int64_t)hq_i * p.q_sh + hh * (D / 2);
  const T* dorow = reinterpret_cast<const T*>(p.d_o) + (int64_t)(q0 + qi) * p.do_sn + (int64_t)hq_i * p.do_sh + hh * (D / 2);
  vec8 qreg[NKS], doreg[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    qreg[ks] = load16<vec8>(qrow + ks * 8);
    doreg[ks] = load16<vec8>(dorow + ks * 8);
  }
  const int64_t stat = (int64_t)hq_i * p.n_tokens + q0 + qi;
  // a row without any visible key has lse = -inf: +inf instead turns every probability of it into 0, not NaN
  const float lse_in = p.lse[stat];
  const float lse_r = lse_in == -INFINITY ? INFINITY : lse_in;
  const float delta_s = p.delta[stat] * p.scale;
  const int jmax = KeyRange<MODE>::hi(p, qi, nc), jmin = KeyRange<MODE>::lo(p, qi);
  const int qi_first = row_lo / p.g, qi_last = (min(rows_total, row_lo + CMP_ROWS) - 1) / p.g;
  const int n_keys = KeyRange<MODE>::hi(p, qi_last, nc) + 1;                 // end of the work-group's key range
  const int jt0 = KeyRange<MODE>::lo(p, qi_first) / CMP_BK * CMP_BK;          // its tile-aligned start

  const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)h * p.k_sh;
  const T* vbase = reinterpret_cast<const T*>(p.v) + (int64_t)h * p.v_sh;
  const uint32_t k_off = kv_tile_offset<T, D>(p.k_sn, tid), v_off = kv_tile_offset<T, D>(p.v_sn, tid);
  const T* ktr = Ks + (4 * hh + ((lane & 15) >> 2)) * KS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  f32x16 dacc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) dacc[dt][i] = 0.f;

  for (int jt = jt0; jt < n_keys; jt += CMP_BK) {
    if (jt != jt0) __syncthreads();
    stage_kv_tile<T, D>(kbase, p.k_sn, k_off, vbase, p.v_sn, v_off, k0 + jt, nc - jt, Ks, Vs, tid);
    __syncthreads();
    f32x16 acc[NA], dp[NA];
#pragma unroll
    for (int a = 0; a < NA; ++a) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        acc[a][i] = 0.f;
        dp[a][i] = 0.f;
      }
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        vec8 kf = load16<vec8>(&Ks[(a * 32 + col) * KS + hh * (D / 2) + ks * 8]);
        acc[a] = Elem<T>::mfma32(kf, qreg[ks], acc[a]);
        vec8 vf = load16<vec8>(&Vs[(a * 32 + col) * VS + hh * (D / 2) + ks * 8]);
        dp[a] = Elem<T>::mfma32(vf, doreg[ks], dp[a]);
      }
    }
    const int limit = jmax - jt, limit_lo = jmin - jt;
    vec8 dsk[NJ];
    // tiles that every row of the wave sees completely need no mask
    if (!__all(limit >= CMP_BK - 1 && limit_lo <= 0)) {
#pragma unroll
      for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = a * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
          if (!(key <= limit && key >= limit_lo)) acc[a][i] = -INFINITY;
        }
    }
    // dS = P (dP - delta) scale
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pv = fast_exp2(acc[a][i] * p.scale_log2 - lse_r);
        dsk[a * 2 + (i >> 3)][i & 7] = (T)(pv * (dp[a][i] * p.scale - delta_s));
      }
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        vec8 kf = lds_read_tr8<T>(ktr + 16 * j * KS + dt * 32, 8 * KS);
        dacc[dt] = Elem<T>::mfma32(kf, dsk[j], dacc[dt]);
      }
  }
  if (!valid) return;
  T* orow = reinterpret_cast<T*>(p.dq) + ((int64_t)(q0 + qi) * (p.g * gridDim.z) + hq_i) * D + 4 * hh;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      vec4 x;
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = (T)dacc[dt][4 * qd + e];
      store8(orow + dt * 32 + 8 * qd, x);
    }
}

template <typename T, int D>
__global__ void __launch_bounds__(256)
cmp_delta_kernel(const T* __restrict__ o, int64_t o_sn, int64_t o_sh, const T* __restrict__ d_o,
                 int64_t do_sn, int64_t do_sh, int64_t n_tokens, int hq, float* __restrict__ delta) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int LPR = D / 8, RPB = 256 / LPR;
  const int64_t R = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
  const int sub = threadIdx.x % LPR;
  if (R >= n_tokens * hq) return;
  const int64_t tok = R / hq;
  const int h = (int)(R - tok * hq);
  vec8 a = load16<vec8>(o + tok * o_sn + (int64_t)h * o_sh + sub * 8);
  vec8 b = load16<vec8>(d_o + tok * do_sn + (int64_t)h * do_sh + sub * 8);
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) s += (float)a[e] * (float)b[e];
#pragma unroll
  for (int o_ = LPR / 2; o_ >= 1; o_ >>= 1) s += __shfl_xor(s, o_, LPR);
  if (sub == 0) delta[(int64_t)h * n_tokens + tok] = s;
}

// work list of the key-major dK/dV kernel: one "block" per tile of 64 compressed keys
__global__ void cmp_kv_blocks_kernel(const int32_t* __restrict__ cu_q, const int32_t* __restrict__ cu_k,
                                     int batch, int hkv, int64_t max_blocks, int kernel_size,
                                     int kernel_stride, int32_t* __restrict__ cu_tiles,
                                     int32_t* __restrict__ counts) {
  __shared__ int total;
  if (threadIdx.x == 0) {
    int acc = 0;
    cu_tiles[0] = 0;
    for (int s = 0; s < batch; ++s) {
      acc += (cu_k[s + 1] - cu_k[s] + CMP_BK - 1) / CMP_BK;
      cu_tiles[s + 1] = acc;
    }
    total = acc;
  }
  __syncthreads();
  for (int64_t gb = threadIdx.x; gb < max_blocks; gb += blockDim.x) {
    int c = 0;
    if (gb < total) {
      const int s = upper_seg(cu_tiles, batch, (int)gb);
      const int q_first = (int)(gb - cu_tiles[s]) * CMP_BK * kernel_stride + kernel_size - 1;
      c = max(0, cu_q[s + 1] - cu_q[s] - q_first);
    }
    for (int h = 0; h < hkv; ++h) counts[h * max_blocks + gb] = c;
  }
}

// work list of the dK/dV kernel in sliding-window mode: one "block" per tile of 64 keys (tokens);
// its rows are the queries from the tile's first key to window tokens past its last key
__global__ void win_kv_blocks_kernel(const int32_t* __restrict__ cu_q, int batch, int hkv, int64_t max_blocks,
                                     int window, int32_t* __restrict__ cu_tiles, int32_t* __restrict__ counts) {
  __shared__ int total;
  if (threadIdx.x == 0) {
    int acc = 0;
    cu_tiles[0] = 0;
    for (int s = 0; s < batch; ++s) {
      acc += (cu_q[s + 1] - cu_q[s] + CMP_BK - 1) / CMP_BK;
      cu_tiles[s + 1] = acc;
    }
    total = acc;
  }
  __syncthreads();
  for (int64_t gb = threadIdx.x; gb < max_blocks; gb += blockDim.x) {
    int c = 0;
    if (gb < total) {
      const int s = upper_seg(cu_tiles, batch, (int)gb);
      const int len = cu_q[s + 1] - cu_q[s];
      const int first = (int)(gb - cu_tiles[s]) * CMP_BK;
      c = max(0, min(len, first + CMP_BK + window) - first);
    }
    for (int h = 0; h < hkv; ++h) counts[h * max_blocks + gb] = c;
  }
}

// ------------------------------------------------------------------ score ----
// score[h, token, j] = 2^(c q[token, h*g] . ck[j, h] - lse[h*g, token]) for visible j
// REBIN (compression window of 2 strides, selection block of 4): the block scores - taps 4 b - 1 .. 4 b + 3 with
// weights 1 2 2 2 1 - are formed in registers and written instead of the per-key probabilities, a quarter of the
// bytes.  A lane holds groups of four consecutive keys, i.e. the last four taps of a block; the first tap is the
// last key of the group before, which the other half of the wave holds (one exchange per group, and one value
// carried over from the previous key tile).
template <typename T, int D, bool REBIN>
__global__ void __launch_bounds__(256)
cmp_score_kernel(CmpParams p) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int KS = CmpLds<D>::KS;
  constexpr int NA = CMP_BK / 32, NKS = D / 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Ks = reinterpret_cast<T*>(smem);

  const int s = blockIdx.y, h = blockIdx.z;
  const int q0 = p.cu_q[s], lq = p.cu_q[s + 1] - q0;
  const int k0 = p.cu_k[s], nc = p.cu_k[s + 1] - k0;
  const int row_lo = blockIdx.x * CMP_ROWS;
  if (row_lo >= lq) return;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int r = row_lo + wv * 32 + col;
  const bool valid = r < lq;
  const int qi = valid ? r : lq - 1;
  const int hq_i = h * p.score_head_step;  // first head of the group (as written: q head = kv head)
  const T* qrow = reinterpret_cast<const T*>(p.q) + (int64_t)(q0 + qi) * p.q_sn + (int64_t)hq_i * p.q_sh + hh * (D / 2);
  vec8 qreg[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) qreg[ks] = load16<vec8>(qrow + ks * 8);
  const float lse_r = p.lse[(int64_t)hq_i * p.n_tokens + q0 + qi];
  int jmax = qi >= p.kernel_size - 1 ? (qi - p.kernel_size + 1) / p.kernel_stride : -1;
  jmax = min(jmax, nc - 1);
  const int qi_last = min(lq, row_lo + CMP_ROWS) - 1;
  const int n_keys = qi_last >= p.kernel_size - 1 ? min(nc, (qi_last - p.kernel_size + 1) / p.kernel_stride + 1) : 0;
  const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)h * p.k_sh;
  float* srow = p.score + ((int64_t)h * p.n_tokens + q0 + qi) * p.score_ld;
  const uint32_t k_off = kv_tile_offset<T, D>(p.k_sn, tid);

  // REBIN: one more tile when the visible keys end on a tile boundary - the block that starts there still owns the
  // last key before it
  const int n_keys_loop = REBIN && n_keys > 0 ? n_keys + 1 : n_keys;
  float carry = 0.f;  // REBIN, lower half of the wave: probability of the key just before this tile
  for (int jt = 0; jt < n_keys_loop; jt += CMP_BK) {
    if (jt) __syncthreads();
    stage_kv_tile<T, D, false>(kbase, p.k_sn, k_off, (const T*)nullptr, 0, 0u, k0 + jt, nc - jt, Ks, (T*)nullptr, tid);
    __syncthreads();
    f32x16 acc[NA];
#pragma unroll
    for (int a = 0; a < NA; ++a) {
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        vec8 kf = load16<vec8>(&Ks[(a * 32 + col) * KS + hh * (D / 2) + ks * 8]);
        acc[a] = Elem<T>::mfma32(kf, qreg[ks], acc[a]);
      }
    }
    const int limit = jmax - jt;
    if constexpr (REBIN) {
      static_assert(NA == 2, "two 32-key halves per tile");
      float x[NA][16], last[NA * 4], recv[NA * 4];
#pragma unroll
      for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = a * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
          x[a][i] = key <= limit ? fast_exp2(acc[a][i] * p.scale_log2 - lse_r) : 0.f;
        }
#pragma unroll
      for (int f = 0; f < NA * 4; ++f) {
        last[f] = x[f >> 2][4 * (f & 3) + 3];
        recv[f] = __shfl_xor(last[f], 32, 64);
      }
#pragma unroll
      for (int f = 0; f < NA * 4; ++f) {
        // the key before this group: the other half's group f (upper half) or f - 1 (lower half)
        const float before = hh ? recv[f] : (f ? recv[f > 0 ? f - 1 : 0] : carry);
        const int a = f >> 2, qd = f & 3;
        float bsum = before;
        bsum += 2.f * x[a][4 * qd];
        bsum += 2.f * x[a][4 * qd + 1];
        bsum += 2.f * x[a][4 * qd + 2];
        bsum += x[a][4 * qd + 3];
        const int blk = jt / 4 + a * 8 + 2 * qd + hh;
        if (valid && blk < p.score_ld) srow[blk] = bsum;
      }
      carry = recv[NA * 4 - 1];
    } else if (valid) {
#pragma unroll
      for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          const int key0 = a * 32 + 8 * qd + 4 * hh;
          if (jt + key0 < p.score_ld) {
            f32x4 x;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              x[e] = key0 + e <= limit ? fast_exp2(acc[a][4 * qd + e] * p.scale_log2 - lse_r) : 0.f;
            *reinterpret_cast<f32x4*>(srow + jt + key0) = x;
          }
        }
    }
  }
}

// ------------------------------------------------------- transform + top-k ----
struct TopkParams {
  const float* score;   // [Hkv, N, score_ld]; only the visible prefix of each row is defined
  int64_t score_ld;
  const int32_t* cu_q;
  const int32_t* cu_k;
  int batch;
  int64_t n_tokens;
  int hkv;
  int kernel_size, kernel_stride, block_size;
  int na, ne;           // kernel_size / kernel_stride, block_size / kernel_stride
  int rebin;            // `score` already holds the block scores before forcing and rounding
  int nblk;             // columns of the block-score matrix: ceil(max_seqlen_q / block_size)
  int t_out;            // min(topk, nblk)
  int init_blocks, local_blocks;
  int to_bf16;
  int32_t* topk_idx;    // [Hkv, N, t_out]
  float* block_score;   // optional [Hkv, N, nblk] fp32 (after the optional bf16 rounding)
};

__device__ __forceinline__ float round_bf16(float x) { return (float)(__bf16)x; }

// One wave per (kv head, query).  NREG > 0 (scores rounded to bf16, at most 64 * NREG blocks): every block score
// is packed with its id into one sortable 32-bit key - bf16 bits above, 0xFFFF - id below, so that the larger
// key is the larger score or, on equal scores, the lower id - and lives in a register; a selection round is a
// plain unsigned maximum over the wave.  NREG == 0: fp32 scores in LDS, (value, id) compared explicitly.
// BIG (more than 64 selected blocks per query, or more blocks than four waves can keep in LDS): one wave per
// work-group, the chosen ids are collected in LDS behind the scores and ranked from there.
template <int NREG, bool BIG = false>
__global__ void __launch_bounds__(BIG ? 64 : 256)
cmp_topk_kernel(TopkParams p) {
  constexpr int WPB = BIG ? 1 : 4;   // waves (= queries) per work-group
  extern __shared__ float bs_all[];  // [WPB waves][nblk] (+ [t_out] ids when BIG), NREG == 0 only
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int h = blockIdx.y;
  const int tok = blockIdx.x * WPB + wv;  // the same for every lane of the wave
  if (tok >= p.n_tokens) return;
  float* bs = bs_all + wv * p.nblk;
  int* sel = reinterpret_cast<int*>(bs_all + p.nblk);  // BIG only
  const int s = upper_seg(p.cu_q, p.batch, tok);
  const int qi = tok - p.cu_q[s];
  const int nc = p.cu_k[s + 1] - p.cu_k[s];
  const int n_vis = qi >= p.kernel_size - 1 ? min(nc, (qi - p.kernel_size + 1) / p.kernel_stride + 1) : 0;
  const int na = p.na, ne = p.ne;
  const int n_off = na + ne - 1, pad = na - 1;
  const int bq = qi / p.block_size;
  const float* srow = p.score + ((int64_t)h * p.n_tokens + tok) * p.score_ld;
  // the usual geometry (compression window of 2 strides, selection block of 4): taps 4 b - 1 .. 4 b + 3 with
  // weights 1 2 2 2 1, four of them one aligned 16-byte load (score rows start 16-byte aligned)
  const bool taps_12221 = na == 2 && ne == 4;
  auto block_score = [&](int b) {
    float acc = 0.f;
    const int c0 = b * ne - pad;
    if (p.rebin) {
      acc = max(4 * b - 1, 0) < n_vis ? srow[b] : 0.f;  // blocks without a visible tap were not written
    } else if (taps_12221) {
      const int c = 4 * b;
      f32x4 x = {0.f, 0.f, 0.f, 0.f};
      if (c + 3 < n_vis) {
        x = *reinterpret_cast<const f32x4*>(srow + c);
      } else {
#pragma unroll
        for (int e = 0; e < 3; ++e)
          if (c + e < n_vis) x[e] = srow[c + e];
      }
      const float xm = (c >= 1 && c - 1 < n_vis) ? srow[c - 1] : 0.f;
      acc = xm;
      acc += 2.f * x[0];
      acc += 2.f * x[1];
      acc += 2.f * x[2];
      acc += x[3];
    } else
    for (int o = 0; o < n_off; ++o) {
      const int c = c0 + o;
      if (c >= 0 && c < n_vis) {
        const int wgt = min(min(o, n_off - 1 - o), min(na, ne) - 1) + 1;
        acc += (float)wgt * srow[c];
      }
    }
    if (b < p.init_blocks || (bq >= b && bq < b + p.local_blocks)) acc = INFINITY;
    if (p.to_bf16) acc = round_bf16(acc);
    if (p.block_score) p.block_score[((int64_t)h * p.n_tokens + tok) * p.nblk + b] = acc;
    return acc;
  };
  int my_id = -1;  // lane t keeps the id chosen in round t
  if (NREG > 0) {
    uint32_t key[NREG > 0 ? NREG : 1];
#pragma unroll
    for (int r = 0; r < NREG; ++r) {
      const int b = lane + 64 * r;
      key[r] = b < p.nblk ? ((__float_as_uint(block_score(b)) >> 16 << 16) | (0xFFFFu - (uint32_t)b)) : 0u;
    }
    for (int t = 0; t < p.t_out; ++t) {
      uint32_t best = key[0];
#pragma unroll
      for (int r = 1; r < NREG; ++r) best = max(best, key[r]);
      best = wave_max_u32(best);
#pragma unroll
      for (int r = 0; r < NREG; ++r) key[r] = key[r] == best ? 0u : key[r];  // keys are distinct
      if (lane == t) my_id = 0xFFFF - (int)(best & 0xFFFFu);
    }
  } else {
    for (int b = lane; b < p.nblk; b += 64) bs[b] = block_score(b);
    __builtin_amdgcn_wave_barrier();
    // t_out rounds of arg-max by (value desc, id asc); taken entries are marked -1 (scores are >= 0)
    for (int t = 0; t < p.t_out; ++t) {
      float best = -2.f;
      int best_id = 0x7fffffff;
      for (int b = lane; b < p.nblk; b += 64) {
        const float vv = bs[b];
        if (vv > best) {
          best = vv;
          best_id = b;
        }
      }
      // scores are >= 0 (or the -2 of a lane without blocks): as 64-bit keys, score bits above and the complement
      // of the id below, the larger key is the larger score or, on equal scores, the lower id
      const uint64_t mine = best < 0.f ? 0ull : ((uint64_t)__float_as_uint(best) << 32) | (0xFFFFFFFFu - (uint32_t)best_id);
      const uint64_t top = wave_max_u64(mine);
      best_id = (int)(0xFFFFFFFFu - (uint32_t)top);
      if (!BIG && lane == t) my_id = best_id;
      if (lane == 0) {
        bs[best_id] = -1.f;
        if (BIG) sel[t] = best_id;
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
  if (BIG) {  // ascending order by rank counting over the list in LDS, then the mask
    for (int i = lane; i < p.t_out; i += 64) {
      const int id = sel[i];
      int rank = 0;
      for (int j = 0; j < p.t_out; ++j) rank += sel[j] < id;
      p.topk_idx[((int64_t)h * p.n_tokens + tok) * p.t_out + rank] = id > bq ? -1 : id;
    }
    return;
  }
  // ascending order by rank counting (ids are distinct), then mask ids above the own block
  const int t_eff = min(p.t_out, 64);
  int rank = 0;
  for (int t = 0; t < t_eff; ++t) {
    const int other = __builtin_amdgcn_readlane(my_id, t);  // uniform lane index: no trip through the LDS crossbar
    if (other < my_id) ++rank;
  }
  if (lane < t_eff)
    p.topk_idx[((int64_t)h * p.n_tokens + tok) * p.t_out + rank] = my_id > bq ? -1 : my_id;
}

// -------------------------------------------------------------- host side ----
template <typename K> static int cmp_set_lds(K kernel, int bytes) {
  if (bytes <= 48 * 1024) return 0;
  hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    set_error("hipFuncSetAttribute(%d B LDS): %s", bytes, hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

struct CmpBwdWs {
  size_t off_delta, off_cu_tiles, off_counts, off_tiles, off_part, total;
  int64_t max_blocks, max_tiles;
};

static CmpBwdWs cmp_bwd_ws(int64_t n, int64_t n_k, int64_t max_q, int batch, int hq, int hkv, int d) {
  CmpBwdWs w;
  const int g = hq / hkv;
  w.max_blocks = (n_k + CMP_BK - 1) / CMP_BK + batch;
  // a key tile is seen by at most max_q queries of its sequence; rows = queries * g
  w.max_tiles = w.max_blocks * ((max_q * g + kv_tile_rows(g) - 1) / kv_tile_rows(g) + 1);
  w.off_delta = 0;
  w.off_cu_tiles = align_up((size_t)n * hq * 4, 256);
  w.off_counts = w.off_cu_tiles + align_up((size_t)(batch + 1) * 4, 256);
  w.off_tiles = w.off_counts + align_up((size_t)hkv * w.max_blocks * 4, 256);
  w.off_part = w.off_tiles + align_up((size_t)hkv * (w.max_blocks + 1) * 4, 256);
  w.total = w.off_part + align_up((size_t)hkv * w.max_tiles * 2 * CMP_BK * d * 4, 256);
  return w;
}

template <typename T, int D, int MODE>
static int attn_fwd_launch(const CmpParams& p, int batch, int hkv, int64_t max_rows, hipStream_t stream) {
  int rc = cmp_set_lds(cmpattn_fwd_kernel<T, D, MODE>, CmpLds<D>::BYTES);
  if (rc) return rc;
  dim3 grid((unsigned)((max_rows + CMP_ROWS - 1) / CMP_ROWS), batch, hkv);
  ProfScope ps_(MODE == CMP_MODE_WINDOW ? "winattn_fwd" : "cmpattn_fwd", stream);
  cmpattn_fwd_kernel<T, D, MODE><<<grid, 256, CmpLds<D>::BYTES, stream>>>(p);
  return 0;
}
template <typename T, int D>
static int cmp_fwd_launch(const CmpParams& p, int batch, int hkv, int64_t max_rows, hipStream_t stream) {
  return attn_fwd_launch<T, D, CMP_MODE_COMPRESSED>(p, batch, hkv, max_rows, stream);
}
template <typename T, int D>
static int win_fwd_launch(const CmpParams& p, int batch, int hkv, int64_t max_rows, hipStream_t stream) {
  return attn_fwd_launch<T, D, CMP_MODE_WINDOW>(p, batch, hkv, max_rows, stream);
}

template <typename T, int D, int MODE>
static int attn_bwd_launch(const CmpParams& p, const SelBwdParams& kv, int batch, int hq, int hkv,
                           int64_t max_rows, int64_t n, hipStream_t stream) {
  constexpr int KVM = MODE == CMP_MODE_WINDOW ? KV_MODE_WINDOW : KV_MODE_COMPRESSED;
  int rc = cmp_set_lds(cmpattn_bwd_dq_kernel<T, D, MODE>, CmpLds<D>::BYTES);
  if (rc) return rc;
  rc = cmp_set_lds(attn_bwd_dkdv_kernel<T, D, CMP_BK, KVM>, KvCfg<D, CMP_BK>::BYTES);
  if (rc) return rc;
  {
    ProfScope ps_(MODE == CMP_MODE_WINDOW ? "winattn_bwd_delta" : "cmpattn_bwd_delta", stream);
    constexpr int RPB = 256 / (D / 8);
    cmp_delta_kernel<T, D><<<(unsigned)((n * hq + RPB - 1) / RPB), 256, 0, stream>>>(
        (const T*)p.o, p.o_sn, p.o_sh, (const T*)p.d_o, p.do_sn, p.do_sh, n, hq, (float*)p.delta);
  }
  {
    ProfScope ps_(MODE == CMP_MODE_WINDOW ? "winattn_bwd_dq" : "cmpattn_bwd_dq", stream);
    dim3 grid((unsigned)((max_rows + CMP_ROWS - 1) / CMP_ROWS), batch, hkv);
    cmpattn_bwd_dq_kernel<T, D, MODE><<<grid, 256, CmpLds<D>::BYTES, stream>>>(p);
  }
  {
    ProfScope ps_(MODE == CMP_MODE_WINDOW ? "winattn_bwd_dkdv" : "cmpattn_bwd_dkdv", stream);
    attn_bwd_dkdv_kernel<T, D, CMP_BK, KVM>
        <<<dim3((unsigned)kv.max_tiles, hkv), KvCfg<D, CMP_BK>::NT, KvCfg<D, CMP_BK>::BYTES, stream>>>(kv);
  }
  {
    ProfScope ps_(MODE == CMP_MODE_WINDOW ? "winattn_bwd_dkdv_reduce" : "cmpattn_bwd_dkdv_reduce", stream);
    attn_bwd_dkdv_reduce_kernel<T, D, CMP_BK, KVM>
        <<<dim3((unsigned)((kv.max_blocks + KV_REDUCE_SPAN - 1) / KV_REDUCE_SPAN), hkv, KV_REDUCE_SPLIT), 256, 0, stream>>>(kv);
  }
  return 0;
}

template <typename T, int D>
static int cmp_bwd_launch(const CmpParams& p, const SelBwdParams& kv, int batch, int hq, int hkv,
                          int64_t max_rows, int64_t n, hipStream_t stream) {
  return attn_bwd_launch<T, D, CMP_MODE_COMPRESSED>(p, kv, batch, hq, hkv, max_rows, n, stream);
}
template <typename T, int D>
static int win_bwd_launch(const CmpParams& p, const SelBwdParams& kv, int batch, int hq, int hkv,
                          int64_t max_rows, int64_t n, hipStream_t stream) {
  return attn_bwd_launch<T, D, CMP_MODE_WINDOW>(p, kv, batch, hq, hkv, max_rows, n, stream);
}

template <typename T, int D>
static int cmp_score_launch(const CmpParams& p, int batch, int hkv, int64_t max_q, hipStream_t stream) {
  ProfScope ps_("cmp_score", stream);
  dim3 grid((unsigned)((max_q + CMP_ROWS - 1) / CMP_ROWS), batch, hkv);
  if (p.rebin) cmp_score_kernel<T, D, true><<<grid, 256, CMP_BK * CmpLds<D>::KS * 2, stream>>>(p);
  else cmp_score_kernel<T, D, false><<<grid, 256, CMP_BK * CmpLds<D>::KS * 2, stream>>>(p);
  return 0;
}

// the lane offsets inside a K / V tile are 32-bit: CMP_BK rows have to span less than 4 GiB
static int cmp_check_strides(int64_t k_sn, int64_t v_sn) {
  const int64_t lim = ((int64_t)1 << 32) / (CMP_BK * 2);
  FSA_CHECK_ARG(k_sn >= 0 && k_sn < lim && v_sn >= 0 && v_sn < lim,
                "compressed / window attention: key or value row stride too large");
  return 0;
}
static int cmp_check_strides(const CmpParams& p) { return cmp_check_strides(p.k_sn, p.v_sn); }

#define FSA_CMP_DISPATCH(FN, P, ...)                                                      \
  do {                                                                                    \
    if (int rc_ = cmp_check_strides(P)) return rc_;                                       \
    if (dtype == FSA_BF16) {                                                              \
      if (head_dim == 64) return FN<__bf16, 64>(P, __VA_ARGS__);                          \
      if (head_dim == 128) return FN<__bf16, 128>(P, __VA_ARGS__);                           \
      if (head_dim == 256) return FN<__bf16, 256>(P, __VA_ARGS__);                           \
    } else {                                                                              \
      if (head_dim == 64) return FN<_Float16, 64>(P, __VA_ARGS__);                           \
      if (head_dim == 128) return FN<_Float16, 128>(P, __VA_ARGS__);                         \
      if (head_dim == 256) return FN<_Float16, 256>(P, __VA_ARGS__);                         \
    }                                                                                     \
    set_error("compressed attention: head_dim=%d not supported (64, 128, 256)", head_dim); \
    return FSA_ERR_UNSUPPORTED;                                                           \
  } while (0)

static int cmp_fwd_dispatch(int dtype, int head_dim, const CmpParams& p, int batch, int hkv,
                            int64_t max_rows, hipStream_t stream) {
  FSA_CMP_DISPATCH(cmp_fwd_launch, p, batch, hkv, max_rows, stream);
}
static int cmp_bwd_dispatch(int dtype, int head_dim, const CmpParams& p, const SelBwdParams& kv, int batch,
                            int hq, int hkv, int64_t max_rows, int64_t n, hipStream_t stream) {
  FSA_CMP_DISPATCH(cmp_bwd_launch, p, kv, batch, hq, hkv, max_rows, n, stream);
}
static int win_fwd_dispatch(int dtype, int head_dim, const CmpParams& p, int batch, int hkv,
                            int64_t max_rows, hipStream_t stream) {
  FSA_CMP_DISPATCH(win_fwd_launch, p, batch, hkv, max_rows, stream);
}
static int win_bwd_dispatch(int dtype, int head_dim, const CmpParams& p, const SelBwdParams& kv, int batch,
                            int hq, int hkv, int64_t max_rows, int64_t n, hipStream_t stream) {
  FSA_CMP_DISPATCH(win_bwd_launch, p, kv, batch, hq, hkv, max_rows, n, stream);
}
static int cmp_score_dispatch(int dtype, int head_dim, const CmpParams& p, int batch, int hkv,
                              int64_t max_q, hipStream_t stream) {
  FSA_CMP_DISPATCH(cmp_score_launch, p, batch, hkv, max_q, stream);
}

}  // namespace fsa

using namespace fsa;

static int cmp_check_common(const char* who, int32_t dtype, int32_t hq, int32_t hkv, int32_t ks,
                            int32_t stride, int32_t batch, int64_t n) {
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "%s: dtype must be bf16 or fp16", who);
  FSA_CHECK_ARG(hkv >= 1 && hq % hkv == 0, "%s: num_q_heads must be a multiple of num_kv_heads", who);
  FSA_CHECK_ARG(ks >= 1 && stride >= 1 && ks % stride == 0,
                "%s: kernel_size must be a positive multiple of kernel_stride", who);
  FSA_CHECK_ARG(batch >= 1 && n >= 1, "%s: empty problem", who);
  return 0;
}

extern "C" int fsa_cmpattn_fwd(const void* q, const void* ck, const void* cv, int32_t dtype,
                               int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n,
                               int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                               const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int32_t batch,
                               int64_t total_q, int64_t max_seqlen_q, int32_t num_q_heads,
                               int32_t num_kv_heads, int32_t head_dim, int32_t kernel_size,
                               int32_t kernel_stride, float softmax_scale, void* o, int64_t o_stride_n,
                               int64_t o_stride_h, float* lse, void* stream_) {
  FSA_CHECK_ARG(q && ck && cv && o && lse && cu_seqlens_q && cu_seqlens_k, "fsa_cmpattn_fwd: null pointer");
  int rc = cmp_check_common("fsa_cmpattn_fwd", dtype, num_q_heads, num_kv_heads, kernel_size, kernel_stride,
                            batch, total_q);
  if (rc) return rc;
  FSA_CHECK_ARG(max_seqlen_q >= 1 && max_seqlen_q <= total_q, "fsa_cmpattn_fwd: bad max_seqlen_q");
  CmpParams p = {};
  p.q = q; p.k = ck; p.v = cv; p.o = o; p.lse = lse;
  p.q_sn = q_stride_n; p.q_sh = q_stride_h; p.k_sn = k_stride_n; p.k_sh = k_stride_h;
  p.v_sn = v_stride_n; p.v_sh = v_stride_h; p.o_sn = o_stride_n; p.o_sh = o_stride_h;
  p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k; p.n_tokens = total_q;
  p.g = num_q_heads / num_kv_heads; p.kernel_size = kernel_size; p.kernel_stride = kernel_stride;
  p.scale = softmax_scale; p.scale_log2 = softmax_scale * LOG2E;
  rc = cmp_fwd_dispatch(dtype, head_dim, p, batch, num_kv_heads, max_seqlen_q * p.g, (hipStream_t)stream_);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_cmpattn_fwd");
  return 0;
}

extern "C" size_t fsa_cmpattn_bwd_workspace_bytes(int64_t total_q, int64_t total_k, int64_t max_seqlen_q,
                                                  int32_t batch, int32_t num_q_heads,
                                                  int32_t num_kv_heads, int32_t head_dim) {
  return cmp_bwd_ws(total_q, total_k, max_seqlen_q, batch, num_q_heads, num_kv_heads, head_dim).total;
}

extern "C" int fsa_cmpattn_bwd(const void* q, const void* ck, const void* cv, const void* o,
                               const void* d_o, const float* lse, int32_t dtype, int64_t q_stride_n,
                               int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                               int64_t v_stride_n, int64_t v_stride_h, int64_t o_stride_n,
                               int64_t o_stride_h, int64_t do_stride_n, int64_t do_stride_h,
                               const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int32_t batch,
                               int64_t total_q, int64_t total_k, int64_t max_seqlen_q,
                               int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                               int32_t kernel_size, int32_t kernel_stride, float softmax_scale, void* dq,
                               void* dck, void* dcv, void* workspace, size_t workspace_bytes,
                               void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(q && ck && cv && o && d_o && lse && dq && dck && dcv && cu_seqlens_q && cu_seqlens_k,
                "fsa_cmpattn_bwd: null pointer");
  int rc = cmp_check_common("fsa_cmpattn_bwd", dtype, num_q_heads, num_kv_heads, kernel_size, kernel_stride,
                            batch, total_q);
  if (rc) return rc;
  FSA_CHECK_ARG(total_k >= 1, "fsa_cmpattn_bwd: no compressed keys");
  FSA_CHECK_ARG(max_seqlen_q >= 1 && max_seqlen_q <= total_q, "fsa_cmpattn_bwd: bad max_seqlen_q");
  CmpBwdWs ws = cmp_bwd_ws(total_q, total_k, max_seqlen_q, batch, num_q_heads, num_kv_heads, head_dim);
  if (!workspace || workspace_bytes < ws.total) {
    set_error("fsa_cmpattn_bwd: workspace too small (%zu < %zu)", workspace_bytes, ws.total);
    return FSA_ERR_WORKSPACE;
  }
  char* wsp = (char*)workspace;
  const int g = num_q_heads / num_kv_heads;
  FSA_CHECK_ARG(kv_qdo_strides_ok(q_stride_n, q_stride_h, do_stride_n, do_stride_h, g, head_dim),
                "fsa_cmpattn_bwd: q / d_o strides too large or negative");
  if (int rc_ = cmp_check_strides(k_stride_n, v_stride_n)) return rc_;
  float* delta = (float*)(wsp + ws.off_delta);
  int32_t* cu_tiles = (int32_t*)(wsp + ws.off_cu_tiles);
  int32_t* counts = (int32_t*)(wsp + ws.off_counts);
  int32_t* tile_prefix = (int32_t*)(wsp + ws.off_tiles);
  cmp_kv_blocks_kernel<<<1, 256, 0, stream>>>(cu_seqlens_q, cu_seqlens_k, batch, num_kv_heads, ws.max_blocks,
                                              kernel_size, kernel_stride, cu_tiles, counts);
  rc = fsa_build_tiles(counts, num_kv_heads, ws.max_blocks, g, kv_tile_rows(g), tile_prefix, stream_);
  if (rc) return rc;

  CmpParams p = {};
  p.q = q; p.k = ck; p.v = cv; p.o = (void*)o; p.d_o = d_o; p.dq = dq; p.lse = (float*)lse; p.delta = delta;
  p.q_sn = q_stride_n; p.q_sh = q_stride_h; p.k_sn = k_stride_n; p.k_sh = k_stride_h;
  p.v_sn = v_stride_n; p.v_sh = v_stride_h; p.o_sn = o_stride_n; p.o_sh = o_stride_h;
  p.do_sn = do_stride_n; p.do_sh = do_stride_h;
  p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k; p.n_tokens = total_q;
  p.g = g; p.kernel_size = kernel_size; p.kernel_stride = kernel_stride;
  p.scale = softmax_scale; p.scale_log2 = softmax_scale * LOG2E;

  SelBwdParams kv = {};
  kv.q = q; kv.k = ck; kv.v = cv; kv.d_o = d_o; kv.lse = lse; kv.delta = delta;
  kv.q_sn = q_stride_n; kv.q_sh = q_stride_h; kv.k_sn = k_stride_n; kv.k_sh = k_stride_h;
  kv.v_sn = v_stride_n; kv.v_sh = v_stride_h; kv.do_sn = do_stride_n; kv.do_sh = do_stride_h;
  kv.cu_seqlens = cu_seqlens_q; kv.cu_blocks = cu_tiles; kv.counts = counts; kv.starts = nullptr;
  kv.sel_tokens = nullptr; kv.tile_prefix = tile_prefix;
  kv.batch = batch; kv.max_blocks = ws.max_blocks; kv.cap = 0; kv.n_tokens = total_q; kv.g = g; kv.g_shift = group_shift(g);
  kv.scale = softmax_scale; kv.scale_log2 = softmax_scale * LOG2E;
  kv.dq_part = nullptr; kv.dkdv_part = (float*)(wsp + ws.off_part); kv.max_tiles = ws.max_tiles;
  kv.kv_tile_rows = kv_tile_rows(g);
  kv.dk = dck; kv.dv = dcv; kv.dk_sn = (int64_t)num_kv_heads * head_dim; kv.dk_sh = head_dim;
  kv.cu_seqlens_k = cu_seqlens_k; kv.kernel_size = kernel_size; kv.kernel_stride = kernel_stride;

  rc = cmp_bwd_dispatch(dtype, head_dim, p, kv, batch, num_q_heads, num_kv_heads, max_seqlen_q * g, total_q,
                        stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_cmpattn_bwd");
  return 0;
}

extern "C" size_t fsa_cmp_topk_workspace_bytes(int64_t total_q, int32_t num_kv_heads, int64_t max_seqlen_k) {
  const int64_t ld = (max_seqlen_k + 3) / 4 * 4;
  return align_up((size_t)total_q * num_kv_heads * ld * 4, 256);
}

extern "C" int fsa_cmp_topk(const void* q, const void* ck, const float* lse, int32_t dtype,
                            int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                            const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int32_t batch,
                            int64_t total_q, int64_t max_seqlen_q, int64_t max_seqlen_k,
                            int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                            int32_t kernel_size, int32_t kernel_stride, int32_t block_size, int32_t topk,
                            int32_t init_blocks, int32_t local_blocks, int32_t scores_to_bf16,
                            int32_t score_head_as_written, float softmax_scale, int32_t* topk_idx,
                            float* block_score, void* workspace,
                            size_t workspace_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(q && ck && lse && topk_idx && cu_seqlens_q && cu_seqlens_k, "fsa_cmp_topk: null pointer");
  int rc = cmp_check_common("fsa_cmp_topk", dtype, num_q_heads, num_kv_heads, kernel_size, kernel_stride,
                            batch, total_q);
  if (rc) return rc;
  FSA_CHECK_ARG(block_size >= kernel_stride && block_size % kernel_stride == 0,
                "fsa_cmp_topk: block_size must be a multiple of kernel_stride");
  FSA_CHECK_ARG(topk >= 1 && max_seqlen_q >= 1 && max_seqlen_k >= 1, "fsa_cmp_topk: bad sizes");
  const int nblk = (int)((max_seqlen_q + block_size - 1) / block_size);
  const int t_out = topk < nblk ? topk : nblk;
  // more than 64 selected blocks per query or more than 4096 blocks per sequence: one-wave work-groups with
  // scores and chosen ids in LDS, which bounds their sum
  const bool big = t_out > 64 || nblk > 4096;
  FSA_CHECK_ARG(!big || ((int64_t)nblk + t_out) * 4 <= 160 * 1024,
                "fsa_cmp_topk: blocks per sequence + selected blocks per query exceed 40960");
  // usual geometry (window of 2 strides, block of 4): the score kernel writes block scores, at most
  // max_seqlen_k / 4 + 1 per query, instead of one probability per compressed key
  const bool rebin = kernel_size == 2 * kernel_stride && block_size == 4 * kernel_stride;
  const int64_t score_cols = rebin ? max_seqlen_k / 4 + 1 : max_seqlen_k;
  const size_t need = fsa_cmp_topk_workspace_bytes(total_q, num_kv_heads, score_cols);
  if (!workspace || workspace_bytes < need) {
    set_error("fsa_cmp_topk: workspace too small (%zu < %zu)", workspace_bytes, need);
    return FSA_ERR_WORKSPACE;
  }
  CmpParams p = {};
  p.q = q; p.k = ck; p.lse = (float*)lse;
  p.q_sn = q_stride_n; p.q_sh = q_stride_h; p.k_sn = k_stride_n; p.k_sh = k_stride_h;
  p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k; p.n_tokens = total_q;
  p.g = num_q_heads / num_kv_heads; p.kernel_size = kernel_size; p.kernel_stride = kernel_stride;
  p.scale = softmax_scale; p.scale_log2 = softmax_scale * LOG2E;
  p.rebin = rebin;
  p.score_head_step = score_head_as_written ? 1 : p.g;
  p.score = (float*)workspace;
  p.score_ld = (score_cols + 3) / 4 * 4;
  rc = cmp_score_dispatch(dtype, head_dim, p, batch, num_kv_heads, max_seqlen_q, stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_cmp_topk score");
  TopkParams tp = {};
  tp.score = p.score; tp.score_ld = p.score_ld; tp.cu_q = cu_seqlens_q; tp.cu_k = cu_seqlens_k;
  tp.batch = batch; tp.n_tokens = total_q; tp.hkv = num_kv_heads;
  tp.kernel_size = kernel_size; tp.kernel_stride = kernel_stride; tp.block_size = block_size;
  tp.na = kernel_size / kernel_stride; tp.ne = block_size / kernel_stride; tp.rebin = p.rebin;
  tp.nblk = nblk; tp.t_out = t_out; tp.init_blocks = init_blocks; tp.local_blocks = local_blocks;
  tp.to_bf16 = scores_to_bf16; tp.topk_idx = topk_idx; tp.block_score = block_score;
  {
    ProfScope ps_("cmp_topk", stream);
    const dim3 grid((unsigned)((total_q + 3) / 4), (unsigned)num_kv_heads);
    if (big) {
      const int lds = (nblk + t_out) * 4;
      rc = cmp_set_lds(cmp_topk_kernel<0, true>, lds);
      if (rc) return rc;
      cmp_topk_kernel<0, true><<<dim3((unsigned)total_q, (unsigned)num_kv_heads), 64, lds, stream>>>(tp);
    } else if (scores_to_bf16 && nblk <= 128) cmp_topk_kernel<2><<<grid, 256, 0, stream>>>(tp);
    else if (scores_to_bf16 && nblk <= 256) cmp_topk_kernel<4><<<grid, 256, 0, stream>>>(tp);
    else if (scores_to_bf16 && nblk <= 512) cmp_topk_kernel<8><<<grid, 256, 0, stream>>>(tp);
    else if (scores_to_bf16 && nblk <= 1024) cmp_topk_kernel<16><<<grid, 256, 0, stream>>>(tp);
    else cmp_topk_kernel<0><<<grid, 256, (size_t)4 * nblk * 4, stream>>>(tp);
  }
  FSA_CHECK_LAUNCH("fsa_cmp_topk select");
  return 0;
}

// ------------------------------------------------------------------------------------------------
// Sliding-window attention (causal band of `window` + 1 keys): the third branch of the module.
extern "C" int fsa_winattn_fwd(const void* q, const void* k, const void* v, int32_t dtype,
                               int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n,
                               int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                               const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens,
                               int64_t max_seqlen, int32_t num_q_heads, int32_t num_kv_heads,
                               int32_t head_dim, int32_t window, float softmax_scale, void* o,
                               int64_t o_stride_n, int64_t o_stride_h, float* lse, void* stream_) {
  FSA_CHECK_ARG(q && k && v && o && lse && cu_seqlens, "fsa_winattn_fwd: null pointer");
  int rc = cmp_check_common("fsa_winattn_fwd", dtype, num_q_heads, num_kv_heads, 1, 1, batch, total_tokens);
  if (rc) return rc;
  FSA_CHECK_ARG(window >= 0 && max_seqlen >= 1 && max_seqlen <= total_tokens, "fsa_winattn_fwd: bad sizes");
  CmpParams p = {};
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
  p.q_sn = q_stride_n; p.q_sh = q_stride_h; p.k_sn = k_stride_n; p.k_sh = k_stride_h;
  p.v_sn = v_stride_n; p.v_sh = v_stride_h; p.o_sn = o_stride_n; p.o_sh = o_stride_h;
  p.cu_q = cu_seqlens; p.cu_k = cu_seqlens; p.n_tokens = total_tokens;
  p.g = num_q_heads / num_kv_heads; p.kernel_size = 1; p.kernel_stride = 1; p.window = window;
  p.scale = softmax_scale; p.scale_log2 = softmax_scale * LOG2E;
  rc = win_fwd_dispatch(dtype, head_dim, p, batch, num_kv_heads, max_seqlen * p.g, (hipStream_t)stream_);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_winattn_fwd");
  return 0;
}

static CmpBwdWs win_bwd_ws(int64_t n, int64_t max_q, int window, int batch, int hq, int hkv, int d) {
  CmpBwdWs w = cmp_bwd_ws(n, n, max_q, batch, hq, hkv, d);
  const int g = hq / hkv;
  const int64_t rows = (int64_t)(CMP_BK + window) * g;
  w.max_tiles = w.max_blocks * ((rows + kv_tile_rows(g) - 1) / kv_tile_rows(g) + 1);
  w.total = w.off_part + align_up((size_t)hkv * w.max_tiles * 2 * CMP_BK * d * 4, 256);
  return w;
}

extern "C" size_t fsa_winattn_bwd_workspace_bytes(int64_t total_tokens, int64_t max_seqlen, int32_t window,
                                                  int32_t batch, int32_t num_q_heads,
                                                  int32_t num_kv_heads, int32_t head_dim) {
  return win_bwd_ws(total_tokens, max_seqlen, window, batch, num_q_heads, num_kv_heads, head_dim).total;
}

extern "C" int fsa_winattn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                               const float* lse, int32_t dtype, int64_t q_stride_n, int64_t q_stride_h,
                               int64_t k_stride_n, int64_t k_stride_h, int64_t v_stride_n,
                               int64_t v_stride_h, int64_t o_stride_n, int64_t o_stride_h,
                               int64_t do_stride_n, int64_t do_stride_h, const int32_t* cu_seqlens,
                               int32_t batch, int64_t total_tokens, int64_t max_seqlen,
                               int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                               int32_t window, float softmax_scale, void* dq, void* dk, void* dv,
                               void* workspace, size_t workspace_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(q && k && v && o && d_o && lse && dq && dk && dv && cu_seqlens, "fsa_winattn_bwd: null pointer");
  int rc = cmp_check_common("fsa_winattn_bwd", dtype, num_q_heads, num_kv_heads, 1, 1, batch, total_tokens);
  if (rc) return rc;
  FSA_CHECK_ARG(window >= 0 && max_seqlen >= 1 && max_seqlen <= total_tokens, "fsa_winattn_bwd: bad sizes");
  CmpBwdWs ws = win_bwd_ws(total_tokens, max_seqlen, window, batch, num_q_heads, num_kv_heads, head_dim);
  if (!workspace || workspace_bytes < ws.total) {
    set_error("fsa_winattn_bwd: workspace too small (%zu < %zu)", workspace_bytes, ws.total);
    return FSA_ERR_WORKSPACE;
  }
  char* wsp = (char*)workspace;
  const int g = num_q_heads / num_kv_heads;
  FSA_CHECK_ARG(kv_qdo_strides_ok(q_stride_n, q_stride_h, do_stride_n, do_stride_h, g, head_dim),
                "fsa_winattn_bwd: q / d_o strides too large or negative");
  if (int rc_ = cmp_check_strides(k_stride_n, v_stride_n)) return rc_;
  float* delta = (float*)(wsp + ws.off_delta);
  int32_t* cu_tiles = (int32_t*)(wsp + ws.off_cu_tiles);
  int32_t* counts = (int32_t*)(wsp + ws.off_counts);
  int32_t* tile_prefix = (int32_t*)(wsp + ws.off_tiles);
  win_kv_blocks_kernel<<<1, 256, 0, stream>>>(cu_seqlens, batch, num_kv_heads, ws.max_blocks, window, cu_tiles,
                                              counts);
  rc = fsa_build_tiles(counts, num_kv_heads, ws.max_blocks, g, kv_tile_rows(g), tile_prefix, stream_);
  if (rc) return rc;

  CmpParams p = {};
  p.q = q; p.k = k; p.v = v; p.o = (void*)o; p.d_o = d_o; p.dq = dq; p.lse = (float*)lse; p.delta = delta;
  p.q_sn = q_stride_n; p.q_sh = q_stride_h; p.k_sn = k_stride_n; p.k_sh = k_stride_h;
  p.v_sn = v_stride_n; p.v_sh = v_stride_h; p.o_sn = o_stride_n; p.o_sh = o_stride_h;
  p.do_sn = do_stride_n; p.do_sh = do_stride_h;
  p.cu_q = cu_seqlens; p.cu_k = cu_seqlens; p.n_tokens = total_tokens;
  p.g = g; p.kernel_size = 1; p.kernel_stride = 1; p.window = window;
  p.scale = softmax_scale; p.scale_log2 = softmax_scale * LOG2E;

  SelBwdParams kv = {};
  kv.q = q; kv.k = k; kv.v = v; kv.d_o = d_o; kv.lse = lse; kv.delta = delta;
  kv.q_sn = q_stride_n; kv.q_sh = q_stride_h; kv.k_sn = k_stride_n; kv.k_sh = k_stride_h;
  kv.v_sn = v_stride_n; kv.v_sh = v_stride_h; kv.do_sn = do_stride_n; kv.do_sh = do_stride_h;
  kv.cu_seqlens = cu_seqlens; kv.cu_blocks = cu_tiles; kv.counts = counts; kv.tile_prefix = tile_prefix;
  kv.batch = batch; kv.max_blocks = ws.max_blocks; kv.n_tokens = total_tokens; kv.g = g; kv.g_shift = group_shift(g);
  kv.scale = softmax_scale; kv.scale_log2 = softmax_scale * LOG2E;
  kv.dkdv_part = (float*)(wsp + ws.off_part); kv.max_tiles = ws.max_tiles; kv.kv_tile_rows = kv_tile_rows(g);
  kv.dk = dk; kv.dv = dv; kv.dk_sn = (int64_t)num_kv_heads * head_dim; kv.dk_sh = head_dim;
  kv.cu_seqlens_k = cu_seqlens; kv.kernel_size = 1; kv.kernel_stride = 1; kv.window = window;

  rc = win_bwd_dispatch(dtype, head_dim, p, kv, batch, num_q_heads, num_kv_heads, max_seqlen * g, total_tokens,
                        stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_winattn_bwd");
  return 0;
}
