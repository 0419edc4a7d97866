// Selected attention backward for gfx950.
//
//   delta    : (lse, sum_d O * dO) pairs [N, Hq]                (HBM stream)
//   dqdkdv   : block-major, contraction over the gathered rows (dkdv_kernel.h
//              with FUSE_DQ).  Each wave owns 16 keys of the block and keeps
//              their K / V fragments in registers; Q / dO tiles of 64 rows go
//              through LDS once and feed S = Q K^T, dP = dO V^T (16x16x32 MFMA)
//              and, through transposing reads, dV^T += dO^T P, dK^T += Q^T dS;
//              dS is exchanged between the waves through LDS and
//              dQ^T = K^T dS^T leaves as one partial dQ row per (query, block,
//              head).  The g heads of a group are rows of the same tile, so
//              dK/dV come out already summed over the group in fp32.  Blocks
//              whose rows span several work-groups write fp32 partials.
//   reduce   : query-major sum of the <= T partial dQ rows, fp32, no atomics;
//              the same launch adds the fp32 dK / dV partials in a fixed order
//
// Formulas: fsa/ops/FSA_topk_sparse_attention.py:1229-1237 (dq),
// :1697-1709 (dk/dv), nsa_ref/ops/topk_sparse_attention.py:197-230 (delta).
#include "fsa_common.h"
#include "dkdv_kernel.h"

namespace fsa {

// ---------------------------------------------------------------- delta ----
template <typename T, int D>
__global__ void __launch_bounds__(256)
selattn_bwd_delta_kernel(const T* __restrict__ o, int64_t o_sn, int64_t o_sh,
                         const T* __restrict__ d_o, int64_t do_sn, int64_t do_sh, int64_t n_tokens,
                         int hq, const float* __restrict__ lse, float2* __restrict__ stat2) {
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
  if (sub == 0) stat2[R] = make_float2(lse[(int64_t)h * n_tokens + tok], s);  // [N, Hq] pairs
}

// Sum of the <= T partial dQ rows of each (query, head).
template <typename T, int D>
__device__ __forceinline__ void dq_reduce_block(const T* __restrict__ dq_part, const int32_t* __restrict__ slot_of,
                                                int64_t cap, int64_t n_tokens, int hq, int g, int topk,
                                                T* __restrict__ dq /* contiguous [N, Hq, D] */, int64_t block) {
  typedef typename Elem<T>::vec8 vec8;
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
  vec8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (T)accv[e];
  store16_stream(dq + (tok * hq + hq_i) * D + sub * 8, out);
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
    dq_reduce_block<T, D>((const T*)a.dq_part, a.slot_of, a.cap, a.n_tokens, a.hq, a.g, a.topk, (T*)a.dq,
                          (int64_t)(b - n_kv));
  }
}

// ------------------------------------------------------------- host side ----
struct BwdWs {
  size_t off_delta, off_dqpart, off_tiles_kv, off_tile_block, off_kvpart, total;
  int64_t max_tiles_kv;
};

static BwdWs bwd_ws_layout(int64_t n, int hq, int hkv, int d, int topk, int bk, int64_t max_blocks) {
  BwdWs w;
  const int g = hq / hkv;
  const size_t cap = (size_t)n * topk;
  w.max_tiles_kv = fsa_max_tiles(n, topk, g, kv_tile_rows(g, d, bk), max_blocks);
  w.off_delta = 0;
  w.off_dqpart = align_up((size_t)n * hq * 8, 256);
  w.off_tiles_kv = w.off_dqpart + align_up(cap * hkv * g * d * 2, 256);
  w.off_tile_block = w.off_tiles_kv + align_up((size_t)hkv * (max_blocks + 1) * 4, 256);
  w.off_kvpart = w.off_tile_block + align_up((size_t)hkv * w.max_tiles_kv * 4, 256);
  w.total = w.off_kvpart + align_up((size_t)hkv * w.max_tiles_kv * 2 * bk * d * 4, 256);
  return w;
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
static int launch_bwd(const SelBwdParams& pkv, int hkv, int64_t tiles_kv, const DqReduceArgs& red,
                      hipStream_t stream) {
  const unsigned kv_spans = (unsigned)((pkv.max_blocks + KV_REDUCE_SPAN - 1) / KV_REDUCE_SPAN);
  int rc = set_lds(attn_bwd_dkdv_kernel<T, D, BK, KV_MODE_SELECTED, true>, KvCfg<D, BK>::BYTES_FUSED);
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

template <typename T>
static int dispatch_bwd(int d, int bk, const SelBwdParams& pkv, int hkv, int64_t tiles_kv,
                        const DqReduceArgs& red, hipStream_t stream) {
#define FSA_CASE(DD, BB) \
  if (d == DD && bk == BB) return launch_bwd<T, DD, BB>(pkv, hkv, tiles_kv, red, stream);
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
static int launch_delta(int d, const void* o, int64_t o_sn, int64_t o_sh, const void* d_o, int64_t do_sn,
                        int64_t do_sh, int64_t n, int hq, const float* lse, float2* stat2, hipStream_t stream) {
  const int64_t rows = n * hq;
#define FSA_CASE(DD)                                                                                     \
  if (d == DD) {                                                                                         \
    constexpr int RPB = 256 / (DD / 8);                                                                  \
    const unsigned grid = (unsigned)((rows + RPB - 1) / RPB);                                            \
    ProfScope ps_("selattn_bwd_delta", stream);                                                          \
    selattn_bwd_delta_kernel<T, DD><<<grid, 256, 0, stream>>>((const T*)o, o_sn, o_sh, (const T*)d_o,    \
                                                              do_sn, do_sh, n, hq, lse, stat2);          \
    return 0;                                                                                            \
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
  float2* stat2 = (float2*)(wsp + ws.off_delta);
  int32_t* tiles_kv = (int32_t*)(wsp + ws.off_tiles_kv);
  int32_t* tile_block = (int32_t*)(wsp + ws.off_tile_block);
  int rc = build_tiles(counts, num_kv_heads, max_blocks, g, kv_tile_rows(g, head_dim, block_size), tiles_kv, tile_block,
                       ws.max_tiles_kv, stream);
  if (rc) return rc;

  const int64_t cap = total_tokens * topk;
  rc = dtype == FSA_BF16
           ? launch_delta<__bf16>(head_dim, o, o_stride_n, o_stride_h, d_o, do_stride_n, do_stride_h,
                                  total_tokens, num_q_heads, lse, stat2, stream)
           : launch_delta<_Float16>(head_dim, o, o_stride_n, o_stride_h, d_o, do_stride_n, do_stride_h,
                                    total_tokens, num_q_heads, lse, stat2, stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_selattn_bwd delta");

  SelBwdParams p;
  p.q = q; p.k = k; p.v = v; p.d_o = d_o; p.lse = lse; p.delta = nullptr; p.stat2 = stat2; p.hq = num_q_heads;
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
  p.tile_prefix = tiles_kv; p.tile_block = tile_block; p.max_tiles = ws.max_tiles_kv; p.kv_tile_rows = kv_tile_rows(g, head_dim, block_size);

  DqReduceArgs red;
  red.dq_part = p.dq_part; red.slot_of = slot_of; red.cap = cap; red.n_tokens = total_tokens;
  red.hq = num_q_heads; red.g = g; red.topk = topk; red.dq = dq;
  rc = dtype == FSA_BF16
           ? dispatch_bwd<__bf16>(head_dim, block_size, p, num_kv_heads, ws.max_tiles_kv, red, stream)
           : dispatch_bwd<_Float16>(head_dim, block_size, p, num_kv_heads, ws.max_tiles_kv, red, stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_selattn_bwd dq/dk/dv");
  return 0;
}
