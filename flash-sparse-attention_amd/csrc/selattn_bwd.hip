// Selected attention backward for gfx950.
//
//   delta    : delta[h, n] = sum_d O * dO                       (HBM stream)
//   dq       : block-major like the forward main kernel.  Per 32 gathered rows
//              S^T = K Q^T, dP^T = V dO^T, dS^T = scale * P^T o (dP^T - delta),
//              dQ^T = K^T dS^T (K^T fragments come from transposing LDS reads);
//              one partial dQ row per (query, block, head)
//   dq_reduce: query-major sum of the <= T partial rows, fp32, no atomics
//   dkdv     : block-major, contraction over the gathered rows.  Each wave owns
//              16 keys of the block and keeps their K / V fragments in
//              registers; Q / dO tiles of 64 rows go through LDS once and feed
//              S = Q K^T, dP = dO V^T (16x16x32 MFMA) and, through transposing
//              reads, dV^T += dO^T P and dK^T += Q^T dS.  The g heads of a
//              group are rows of the same tile, so dK/dV come out already summed
//              over the group in fp32.  Blocks whose rows span several
//              work-groups write fp32 partials that dkdv_reduce adds in a fixed
//              order.
//
// Formulas: fsa/ops/FSA_topk_sparse_attention.py:1229-1237 (dq),
// :1697-1709 (dk/dv), nsa_ref/ops/topk_sparse_attention.py:197-230 (delta).
#include "fsa_common.h"
#include "dkdv_kernel.h"

#include <stdlib.h>

namespace fsa {

// ---------------------------------------------------------------- delta ----
template <typename T, int D>
__global__ void __launch_bounds__(256)
selattn_bwd_delta_kernel(const T* __restrict__ o, int64_t o_sn, int64_t o_sh,
                         const T* __restrict__ d_o, int64_t do_sn, int64_t do_sh, int64_t n_tokens,
                         int hq, float* __restrict__ delta) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int LPR = D / 8, RPB = 256 / LPR;
  const int64_t R = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
  const int sub = threadIdx.x % LPR;
  if (R >= n_tokens * hq) return;
  const int64_t tok = R / hq;
  const int h = (int)(R - tok * hq);
  vec8 a = load16_stream<vec8>(o + tok * o_sn + (int64_t)h * o_sh + sub * 8);
  vec8 b = load16<vec8>(d_o + tok * do_sn + (int64_t)h * do_sh + sub * 8);
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) s += (float)a[e] * (float)b[e];
#pragma unroll
  for (int o_ = LPR / 2; o_ >= 1; o_ >>= 1) s += __shfl_xor(s, o_, LPR);
  if (sub == 0) delta[(int64_t)h * n_tokens + tok] = s;
}

// ------------------------------------------------------------------- dq ----
constexpr int DQ_THREADS = 256;
constexpr int DQ_WG_ROWS = 128;
constexpr int DQ_TILE_ROWS = 8 * DQ_WG_ROWS;

template <int D, int BK> struct DqLds {
  static constexpr int KS = D + 8;
  static constexpr int VS = D + 8;
  static constexpr int BYTES = (BK * KS + BK * VS) * 2;
  static constexpr int MIN_WAVES = (D <= 128 && BK <= 64) ? 2 : 1;
};

template <typename T, int D, int BK>
__global__ void __launch_bounds__(DQ_THREADS, (DqLds<D, BK>::MIN_WAVES))
selattn_bwd_dq_kernel(SelBwdParams p) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int KS = DqLds<D, BK>::KS, VS = DqLds<D, BK>::VS;
  constexpr int NA = BK / 32, NKS = D / 16, NDT = D / 32, NJ = BK / 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Ks = reinterpret_cast<T*>(smem);
  T* Vs = Ks + BK * KS;

  const int h = blockIdx.y;
  const int64_t nbp1 = p.max_blocks + 1;
  const int32_t* tp = p.tile_prefix + h * nbp1;
  const int w = blockIdx.x;
  if (w >= tp[p.max_blocks]) return;
  const int gb = upper_seg(tp, (int)p.max_blocks, w);
  const int s = upper_seg(p.cu_blocks, p.batch, gb);
  const int b_local = gb - p.cu_blocks[s];
  const int seq_start = p.cu_seqlens[s], seq_end = p.cu_seqlens[s + 1];
  const int tok0 = seq_start + b_local * BK;
  const int rows = p.counts[h * p.max_blocks + gb] * p.g;
  const int start = p.starts[h * nbp1 + gb];
  const int row_lo = (w - tp[gb]) * DQ_TILE_ROWS;
  const int row_hi = min(rows, row_lo + DQ_TILE_ROWS);

  const int tid = threadIdx.x;
  const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)h * p.k_sh;
  const T* vbase = reinterpret_cast<const T*>(p.v) + (int64_t)h * p.v_sh;
  for (int c = tid; c < BK * (D / 8); c += DQ_THREADS) {
    const int row = c / (D / 8), col = c % (D / 8);
    const int tok = tok0 + row;
    vec8 x = zero8<T>(), y = zero8<T>();
    if (tok < seq_end) {
      x = load16<vec8>(kbase + (int64_t)tok * p.k_sn + col * 8);
      y = load16<vec8>(vbase + (int64_t)tok * p.v_sn + col * 8);
    }
    store16(&Ks[row * KS + col * 8], x);
    store16(&Vs[row * VS + col * 8], y);
  }
  __syncthreads();

  const int lane = tid & 63, wv = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int32_t* toks = p.sel_tokens + (int64_t)h * p.cap + start;
  const T* qbase = reinterpret_cast<const T*>(p.q) + (int64_t)h * p.g * p.q_sh + hh * (D / 2);
  const T* dobase = reinterpret_cast<const T*>(p.d_o) + (int64_t)h * p.g * p.do_sh + hh * (D / 2);
  const int64_t prow0 = ((int64_t)h * p.cap + start) * p.g;
  T* dqpart = reinterpret_cast<T*>(p.dq_part);
  const T* ktr = Ks + (4 * hh + ((lane & 15) >> 2)) * KS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  for (int sub = row_lo + wv * 32; sub < row_hi; sub += DQ_WG_ROWS) {
    const int r = sub + col;
    const bool valid = r < row_hi;
    const int rr = valid ? r : row_hi - 1;
    const int trank = div_group(rr, p.g, p.g_shift);
    const int head = rr - trank * p.g;
    const int token = toks[trank];
    const T* qrow = qbase + (int64_t)token * p.q_sn + (int64_t)head * p.q_sh;
    const T* dorow = dobase + (int64_t)token * p.do_sn + (int64_t)head * p.do_sh;
    vec8 qreg[NKS], doreg[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) qreg[ks] = load16<vec8>(qrow + ks * 8);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) doreg[ks] = load16<vec8>(dorow + ks * 8);
    const int64_t stat = (int64_t)(h * p.g + head) * p.n_tokens + token;
    const float lse_r = p.lse[stat];
    const float delta_r = p.delta[stat];

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
    const int limit = (token - seq_start) - b_local * BK;
    vec8 dsk[NJ];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = a * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
        const float pv = key <= limit ? fast_exp2(acc[a][i] * p.scale_log2 - lse_r) : 0.f;
        const float ds = pv * (dp[a][i] - delta_r) * p.scale;
        dsk[a * 2 + (i >> 3)][i & 7] = (T)ds;
      }
    T* orow = dqpart + (prow0 + r) * D + hh * (D / 2);
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      f32x16 dacc;
#pragma unroll
      for (int i = 0; i < 16; ++i) dacc[i] = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        vec8 kf = lds_read_tr8<T>(ktr + 16 * j * KS + dt * 32, 8 * KS);
        dacc = Elem<T>::mfma32(kf, dsk[j], dacc);
      }
      if (valid) {
#pragma unroll
        for (int c8 = 0; c8 < 2; ++c8) {
          vec8 x;
#pragma unroll
          for (int e = 0; e < 8; ++e) x[e] = (T)dacc[c8 * 8 + e];
          store16(orow + dt * 16 + c8 * 8, x);
        }
      }
    }
  }
}

// Sum of the <= T partial dQ rows of each (query, head); undoes the lane-native order.
template <typename T, int D>
__device__ __forceinline__ void dq_reduce_block(const T* __restrict__ dq_part, const int32_t* __restrict__ slot_of,
                                                int64_t cap, int64_t n_tokens, int hq, int g, int topk, int natural,
                                                T* __restrict__ dq /* contiguous [N, Hq, D] */, int64_t block) {
  typedef typename Elem<T>::vec8 vec8;
  typedef typename Elem<T>::vec4 vec4;
  constexpr int LPR = D / 8, RPB = 256 / LPR;
  const int64_t R = block * RPB + threadIdx.x / LPR;
  const int sub = threadIdx.x % LPR;
  if (R >= n_tokens * hq) return;
  const int64_t tok = R / hq;
  const int hq_i = (int)(R - tok * hq);
  const int kh = hq_i / g, head = hq_i - kh * g;
  const int32_t* so = slot_of + ((int64_t)kh * n_tokens + tok) * topk;
  float accv[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) accv[e] = 0.f;
  // the LPR lanes of a row split the slots: a slot's position is loaded once by its owner and handed round by
  // shuffles, so the row loads of a chunk of LPR slots are independent of each other
  for (int t0 = 0; t0 < topk; t0 += LPR) {
    const int pidx_mine = t0 + sub < topk ? so[t0 + sub] : -1;
#pragma unroll
    for (int j = 0; j < LPR; ++j) {
      const int pidx = __shfl(pidx_mine, j, LPR);
      if (pidx >= 0) {
        const int64_t prow = ((int64_t)kh * cap + pidx) * g + head;
        vec8 x = load16_stream<vec8>(dq_part + prow * D + sub * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) accv[e] += (float)x[e];
      }
    }
  }
  if (natural) {  // partial rows written by the fused kernel are in plain d order
    vec8 out;
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = (T)accv[e];
    store16_stream(dq + (tok * hq + hq_i) * D + sub * 8, out);
    return;
  }
  const int pos = sub * 8;
  const int hh = pos / (D / 2), rem = pos % (D / 2);
  const int dt = rem / 16, i0 = rem % 16;
  T* orow = dq + (tok * hq + hq_i) * D + dt * 32 + 4 * hh + 8 * (i0 >> 2);
  vec4 a, b;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    a[e] = (T)accv[e];
    b[e] = (T)accv[4 + e];
  }
  store8(orow, a);
  store8(orow + 8, b);
}

template <typename T, int D>
__global__ void __launch_bounds__(256)
selattn_bwd_dq_reduce_kernel(const T* __restrict__ dq_part, const int32_t* __restrict__ slot_of,
                             int64_t cap, int64_t n_tokens, int hq, int g, int topk, int natural,
                             T* __restrict__ dq) {
  dq_reduce_block<T, D>(dq_part, slot_of, cap, n_tokens, hq, g, topk, natural, dq, blockIdx.x);
}

// The two reductions that end the fused backward in one launch: the first n_kv work-groups add up the fp32 dK / dV
// partials of the blocks that were shared by several work-groups (few, and latency bound), the others the partial
// dQ rows, so the small reduction runs in the shadow of the large one instead of after it.
struct DqReduceArgs {
  const void* dq_part;
  const int32_t* slot_of;
  int64_t cap, n_tokens;
  int hq, g, topk;
  void* dq;
};
template <typename T, int D, int BK>
__global__ void __launch_bounds__(256)
selattn_bwd_reduce_kernel(SelBwdParams p, DqReduceArgs a, int n_kv, int hkv) {
  const int b = blockIdx.x;
  if (b < n_kv) {
    const int bz = b % KV_REDUCE_SPLIT, h = (b / KV_REDUCE_SPLIT) % hkv, bx = b / (KV_REDUCE_SPLIT * hkv);
    dkdv_reduce_block<T, D, BK, KV_MODE_SELECTED, 4>(p, bx, h, bz, KV_REDUCE_SPLIT);
  } else {
    dq_reduce_block<T, D>((const T*)a.dq_part, a.slot_of, a.cap, a.n_tokens, a.hq, a.g, a.topk, 1, (T*)a.dq,
                          (int64_t)(b - n_kv));
  }
}

// ------------------------------------------------------------- host side ----
struct BwdWs {
  size_t off_delta, off_dqpart, off_tiles_dq, off_tiles_kv, off_kvpart, total;
  int64_t max_tiles_dq, max_tiles_kv;
};

static BwdWs bwd_ws_layout(int64_t n, int hq, int hkv, int d, int topk, int bk, int64_t max_blocks) {
  BwdWs w;
  const int g = hq / hkv;
  const size_t cap = (size_t)n * topk;
  w.max_tiles_dq = fsa_max_tiles(n, topk, g, DQ_TILE_ROWS, max_blocks);
  w.max_tiles_kv = fsa_max_tiles(n, topk, g, kv_tile_rows(g, d, bk), max_blocks);
  w.off_delta = 0;
  w.off_dqpart = align_up((size_t)n * hq * 4, 256);
  w.off_tiles_dq = w.off_dqpart + align_up(cap * hkv * g * d * 2, 256);
  w.off_tiles_kv = w.off_tiles_dq + align_up((size_t)hkv * (max_blocks + 1) * 4, 256);
  w.off_kvpart = w.off_tiles_kv + align_up((size_t)hkv * (max_blocks + 1) * 4, 256);
  w.total = w.off_kvpart + align_up((size_t)hkv * w.max_tiles_kv * 2 * bk * d * 4, 256);
  return w;
}

// FSA_BWD_SPLIT=1 selects the two-kernel backward (separate dQ and dK/dV kernels, each
// gathering Q and dO); the default is the fused kernel.  Read once.
static bool fused_dq() {
  static const bool v = [] {
    const char* e = getenv("FSA_BWD_SPLIT");
    return !(e && e[0] == '1');
  }();
  return v;
}

template <typename K> static int set_lds(K kernel, int bytes) {
  if (bytes <= 48 * 1024) return 0;
  hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    set_error("hipFuncSetAttribute(%d B LDS): %s", bytes, hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

template <typename T, int D, int BK>
static int launch_bwd(const SelBwdParams& pdq, const SelBwdParams& pkv, int hkv, int64_t tiles_dq,
                      int64_t tiles_kv, const DqReduceArgs& red, hipStream_t stream) {
  int rc = 0;
  const unsigned kv_spans = (unsigned)((pkv.max_blocks + KV_REDUCE_SPAN - 1) / KV_REDUCE_SPAN);
  if (fused_dq()) {
    rc = set_lds(attn_bwd_dkdv_kernel<T, D, BK, KV_MODE_SELECTED, true>, KvCfg<D, BK>::BYTES_FUSED);
    if (rc) return rc;
    {
      ProfScope ps_("selattn_bwd_dqdkdv", stream);
      attn_bwd_dkdv_kernel<T, D, BK, KV_MODE_SELECTED, true>
          <<<dim3((unsigned)tiles_kv, hkv), KvCfg<D, BK>::NT, KvCfg<D, BK>::BYTES_FUSED, stream>>>(pkv);
    }
    constexpr int RPB = 256 / (D / 8);
    const int64_t rows = red.n_tokens * red.hq;
    const int64_t n_kv = (int64_t)kv_spans * hkv * KV_REDUCE_SPLIT, n_dq = (rows + RPB - 1) / RPB;
    ProfScope ps_("selattn_bwd_dq_reduce", stream);
    selattn_bwd_reduce_kernel<T, D, BK><<<(unsigned)(n_kv + n_dq), 256, 0, stream>>>(pkv, red, (int)n_kv, hkv);
    return 0;
  }
  rc = set_lds(selattn_bwd_dq_kernel<T, D, BK>, DqLds<D, BK>::BYTES);
  if (rc) return rc;
  rc = set_lds(attn_bwd_dkdv_kernel<T, D, BK, KV_MODE_SELECTED>, KvCfg<D, BK>::BYTES);
  if (rc) return rc;
  {
    ProfScope ps_("selattn_bwd_dq", stream);
    selattn_bwd_dq_kernel<T, D, BK><<<dim3((unsigned)tiles_dq, hkv), DQ_THREADS, DqLds<D, BK>::BYTES, stream>>>(pdq);
  }
  {
    ProfScope ps_("selattn_bwd_dkdv", stream);
    attn_bwd_dkdv_kernel<T, D, BK, KV_MODE_SELECTED><<<dim3((unsigned)tiles_kv, hkv), KvCfg<D, BK>::NT, KvCfg<D, BK>::BYTES, stream>>>(pkv);
  }
  {
    ProfScope ps_("selattn_bwd_dkdv_reduce", stream);
    attn_bwd_dkdv_reduce_kernel<T, D, BK, KV_MODE_SELECTED><<<dim3(kv_spans, hkv, KV_REDUCE_SPLIT), 256, 0, stream>>>(pkv);
  }
  return 0;
}

template <typename T>
static int dispatch_bwd(int d, int bk, const SelBwdParams& pdq, const SelBwdParams& pkv, int hkv,
                        int64_t tiles_dq, int64_t tiles_kv, const DqReduceArgs& red, hipStream_t stream) {
#define FSA_CASE(DD, BB) \
  if (d == DD && bk == BB) return launch_bwd<T, DD, BB>(pdq, pkv, hkv, tiles_dq, tiles_kv, red, stream);
  FSA_CASE(128, 64)
  FSA_CASE(128, 32)
  FSA_CASE(128, 128)
  FSA_CASE(64, 32)
  FSA_CASE(64, 64)
  FSA_CASE(64, 128)
  FSA_CASE(256, 32)
  FSA_CASE(256, 64)
  FSA_CASE(256, 128)
#undef FSA_CASE
  set_error("selected attention backward: head_dim=%d with block_size=%d is not supported "
            "(head_dim in {64,128,256}, block_size in {32,64,128})", d, bk);
  return FSA_ERR_UNSUPPORTED;
}

template <typename T>
static int launch_rowwise(int d, const void* o, int64_t o_sn, int64_t o_sh, const void* d_o,
                          int64_t do_sn, int64_t do_sh, int64_t n, int hq, float* delta,
                          const void* dq_part, const int32_t* slot_of, int64_t cap, int g, int topk,
                          void* dq, bool second, hipStream_t stream) {
  const int64_t rows = n * hq;
#define FSA_CASE(DD)                                                                               \
  if (d == DD) {                                                                                   \
    constexpr int RPB = 256 / (DD / 8);                                                            \
    const unsigned grid = (unsigned)((rows + RPB - 1) / RPB);                                      \
    ProfScope ps_(second ? "selattn_bwd_dq_reduce" : "selattn_bwd_delta", stream);                 \
    if (!second)                                                                                   \
      selattn_bwd_delta_kernel<T, DD><<<grid, 256, 0, stream>>>((const T*)o, o_sn, o_sh,           \
                                                                (const T*)d_o, do_sn, do_sh, n, hq, \
                                                                delta);                            \
    else                                                                                           \
      selattn_bwd_dq_reduce_kernel<T, DD><<<grid, 256, 0, stream>>>((const T*)dq_part, slot_of, cap, \
                                                                    n, hq, g, topk,                \
                                                                    fused_dq() ? 1 : 0, (T*)dq);   \
    return 0;                                                                                      \
  }
  FSA_CASE(64)
  FSA_CASE(128)
  FSA_CASE(256)
#undef FSA_CASE
  set_error("selected attention backward: head_dim=%d not supported", d);
  return FSA_ERR_UNSUPPORTED;
}

}  // namespace fsa

using namespace fsa;

extern "C" size_t fsa_selattn_bwd_workspace_bytes(int64_t total_tokens, int32_t num_q_heads,
                                                  int32_t num_kv_heads, int32_t head_dim, int32_t topk,
                                                  int32_t block_size, int64_t max_blocks) {
  return bwd_ws_layout(total_tokens, num_q_heads, num_kv_heads, head_dim, topk, block_size, max_blocks)
      .total;
}

extern "C" int fsa_selattn_bwd(const void* q, const void* k, const void* v, const void* o,
                               const void* d_o, const float* lse, int32_t dtype, int64_t q_stride_n,
                               int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                               int64_t v_stride_n, int64_t v_stride_h, int64_t o_stride_n,
                               int64_t o_stride_h, int64_t do_stride_n, int64_t do_stride_h,
                               const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens,
                               int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                               int32_t topk, int32_t block_size, int64_t max_blocks,
                               float softmax_scale, const int32_t* cu_blocks, const int32_t* counts,
                               const int32_t* starts, const int32_t* sel_tokens,
                               const int32_t* slot_of, void* dq, void* dk, void* dv, void* workspace,
                               size_t workspace_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(q && k && v && o && d_o && lse && dq && dk && dv && cu_seqlens && cu_blocks && counts &&
                    starts && sel_tokens && slot_of, "fsa_selattn_bwd: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_selattn_bwd: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(num_kv_heads >= 1 && num_q_heads % num_kv_heads == 0,
                "fsa_selattn_bwd: num_q_heads must be a multiple of num_kv_heads");
  FSA_CHECK_ARG(batch >= 1 && total_tokens >= 1 && topk >= 1, "fsa_selattn_bwd: empty problem");
  FSA_CHECK_ARG(total_tokens * topk < ((int64_t)1 << 31), "fsa_selattn_bwd: total_tokens*topk >= 2^31");
  FSA_CHECK_ARG((q_stride_n | q_stride_h | k_stride_n | k_stride_h | v_stride_n | v_stride_h |
                 o_stride_n | o_stride_h | do_stride_n | do_stride_h) % 8 == 0,
                "fsa_selattn_bwd: strides must be multiples of 8 elements (16-byte rows)");
  const int g = num_q_heads / num_kv_heads;
  FSA_CHECK_ARG(kv_qdo_strides_ok(q_stride_n, q_stride_h, do_stride_n, do_stride_h, g, head_dim),
                "fsa_selattn_bwd: q / d_o strides too large or negative");
  BwdWs ws = bwd_ws_layout(total_tokens, num_q_heads, num_kv_heads, head_dim, topk, block_size, max_blocks);
  if (!workspace || workspace_bytes < ws.total) {
    set_error("fsa_selattn_bwd: workspace too small (%zu < %zu)", workspace_bytes, ws.total);
    return FSA_ERR_WORKSPACE;
  }
  char* wsp = (char*)workspace;
  float* delta = (float*)(wsp + ws.off_delta);
  int32_t* tiles_dq = (int32_t*)(wsp + ws.off_tiles_dq);
  int32_t* tiles_kv = (int32_t*)(wsp + ws.off_tiles_kv);
  int rc = 0;
  if (!fused_dq()) {  // the tile list of the separate dQ kernel
    rc = fsa_build_tiles(counts, num_kv_heads, max_blocks, g, DQ_TILE_ROWS, tiles_dq, stream_);
    if (rc) return rc;
  }
  rc = fsa_build_tiles(counts, num_kv_heads, max_blocks, g, kv_tile_rows(g, head_dim, block_size), tiles_kv, stream_);
  if (rc) return rc;

  const int64_t cap = total_tokens * topk;
  rc = dtype == FSA_BF16
           ? launch_rowwise<__bf16>(head_dim, o, o_stride_n, o_stride_h, d_o, do_stride_n, do_stride_h,
                                    total_tokens, num_q_heads, delta, nullptr, nullptr, cap, g, topk,
                                    nullptr, false, stream)
           : launch_rowwise<_Float16>(head_dim, o, o_stride_n, o_stride_h, d_o, do_stride_n,
                                      do_stride_h, total_tokens, num_q_heads, delta, nullptr, nullptr,
                                      cap, g, topk, nullptr, false, stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_selattn_bwd delta");

  SelBwdParams p;
  p.q = q; p.k = k; p.v = v; p.d_o = d_o; p.lse = lse; p.delta = delta;
  p.q_sn = q_stride_n; p.q_sh = q_stride_h; p.k_sn = k_stride_n; p.k_sh = k_stride_h;
  p.v_sn = v_stride_n; p.v_sh = v_stride_h; p.do_sn = do_stride_n; p.do_sh = do_stride_h;
  p.cu_seqlens = cu_seqlens; p.cu_blocks = cu_blocks; p.counts = counts; p.starts = starts;
  p.sel_tokens = sel_tokens;
  p.batch = batch; p.max_blocks = max_blocks; p.cap = cap; p.n_tokens = total_tokens; p.g = g; p.g_shift = group_shift(g);
  p.scale = softmax_scale; p.scale_log2 = softmax_scale * LOG2E;
  p.dq_part = wsp + ws.off_dqpart;
  p.dkdv_part = (float*)(wsp + ws.off_kvpart);
  p.dk = dk; p.dv = dv;
  p.dk_sn = (int64_t)num_kv_heads * head_dim; p.dk_sh = head_dim;
  p.cu_seqlens_k = nullptr; p.kernel_size = 0; p.kernel_stride = 1;
  SelBwdParams pdq = p, pkv = p;
  pdq.tile_prefix = tiles_dq; pdq.max_tiles = ws.max_tiles_dq; pdq.kv_tile_rows = 0;
  pkv.tile_prefix = tiles_kv; pkv.max_tiles = ws.max_tiles_kv; pkv.kv_tile_rows = kv_tile_rows(g, head_dim, block_size);

  DqReduceArgs red;
  red.dq_part = p.dq_part; red.slot_of = slot_of; red.cap = cap; red.n_tokens = total_tokens;
  red.hq = num_q_heads; red.g = g; red.topk = topk; red.dq = dq;
  rc = dtype == FSA_BF16
           ? dispatch_bwd<__bf16>(head_dim, block_size, pdq, pkv, num_kv_heads, ws.max_tiles_dq,
                                  ws.max_tiles_kv, red, stream)
           : dispatch_bwd<_Float16>(head_dim, block_size, pdq, pkv, num_kv_heads, ws.max_tiles_dq,
                                    ws.max_tiles_kv, red, stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_selattn_bwd dq/dkdv");
  if (!fused_dq()) {  // the fused path ends with the combined reduction launched above
    rc = dtype == FSA_BF16
             ? launch_rowwise<__bf16>(head_dim, nullptr, 0, 0, nullptr, 0, 0, total_tokens, num_q_heads,
                                      nullptr, p.dq_part, slot_of, cap, g, topk, dq, true, stream)
             : launch_rowwise<_Float16>(head_dim, nullptr, 0, 0, nullptr, 0, 0, total_tokens, num_q_heads,
                                        nullptr, p.dq_part, slot_of, cap, g, topk, dq, true, stream);
    if (rc) return rc;
  }
  FSA_CHECK_LAUNCH("fsa_selattn_bwd dq reduce");
  return 0;
}
