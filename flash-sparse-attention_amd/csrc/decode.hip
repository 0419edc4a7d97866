// One-step decode for gfx950: one new query per request against its caches.
//
//   decode_attn_kernel (compressed mode): the g heads of a kv group attend every
//       visible compressed key of the request; the raw scores of one "scoring"
//       head are kept for the block selection.
//   decode_attn_kernel (selected mode): the g heads attend the cached keys of
//       the T selected blocks.
//   decode_topk_kernel: probabilities -> re-binned block scores -> top-k ids.
//
// Both attention modes are HBM-bound streams of K/V rows (g rows of queries
// only).  The keys of a (request, kv head) are split over work-groups of 512
// keys so that the grid fills the chip whatever the cache lengths are; inside a
// work-group the four waves take 32-key tiles round-robin: K fragments go
// straight from global memory into 16x16x32 MFMA operands, the V tile is staged
// in a wave-private LDS region and read back transposed.  The kernel is kept
// lean in registers (several waves per SIMD keep enough loads in flight).  The
// waves' partial (m, l, O) are merged through LDS into one fp32 partial per
// work-group; a small merge kernel combines the partials of a request in a fixed
// order.  The query heads occupy the first g of the 16 MFMA columns; column g
// carries the scoring head.
//
// Semantics: fsa_preview/ops/compressed_attention_decode.py:361-490 (attention),
// :494-592 (scores), :284-357 (transform), :203-205 (top-k);
// fsa_preview/ops/selected_attention_decode.py:8-42.
#include "fsa_common.h"

namespace fsa {

constexpr int DEC_MODE_COMPRESSED = 0;
constexpr int DEC_MODE_SELECTED = 1;
constexpr int DEC_TK = 32;    // keys per wave tile
constexpr int DEC_TPS = 16;   // tiles per work-group (512 keys)

struct DecParams {
  const void* q;   // [B, Hq, D]
  const void* k;   // [total, Hkv, D]
  const void* v;
  int64_t q_sb, q_sh, k_sn, k_sh, v_sn, v_sh;
  const int32_t* cu_k;      // [B+1] rows of k / v per request
  const int32_t* pos;       // compressed mode: position of the query
  const int32_t* topk_idx;  // selected mode: [Hkv, B, T]
  int batch, hq, hkv, g, topk, block_size, kernel_size, kernel_stride;
  float scale_log2;
  void* o;                  // [B, Hq, D] contiguous
  float* lse;               // [Hq, B]
  float* raw_score;         // compressed mode, optional: [Hkv, B, raw_ld] unscaled q.k of the scoring head
  int64_t raw_ld;
  int score_head_as_written;  // 0: first head of the group, 1: q-head with the kv head's own index
  int max_keys;             // compressed mode: host upper bound of the visible keys of a request (more are ignored)
  float* part;              // [B, Hkv, nsplit, g, 2 + D]: base-2 scaled max, sum, unnormalised O
  int nsplit;
};

template <int D> struct DecLds {
  static constexpr int VS = D + 8;
  static constexpr int WAVE_BYTES = DEC_TK * VS * 2;
  static constexpr int MERGE_BYTES = 4 * (D * 16 + 32) * 4;
  static constexpr int BYTES = 4 * WAVE_BYTES > MERGE_BYTES ? 4 * WAVE_BYTES : MERGE_BYTES;
};

// number of 32-key tiles of request b (and, in compressed mode, its visible keys)
template <int MODE>
__device__ __forceinline__ int dec_tiles(const DecParams& p, int b, int len, int& n_keys, int& tpb) {
  n_keys = 0;
  tpb = 1;
  if (MODE == DEC_MODE_COMPRESSED) {
    const int qp = p.pos[b];
    n_keys = qp >= p.kernel_size - 1 ? min(len, (qp - p.kernel_size + 1) / p.kernel_stride + 1) : 0;
    n_keys = min(n_keys, p.max_keys);
    return (n_keys + DEC_TK - 1) / DEC_TK;
  }
  tpb = (p.block_size + DEC_TK - 1) / DEC_TK;
  return p.topk * tpb;
}

template <typename T, int D, int MODE>
__global__ void __launch_bounds__(256, 2)
decode_attn_kernel(DecParams p) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int VS = DecLds<D>::VS;
  constexpr int NS = D / 32, NDT = D / 16, VCH = DEC_TK * (D / 8) / 64;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // kv heads vary fastest over the grid: work-groups that run together read neighbouring 2*D-byte pieces of the
  // same cache rows
  const int h = blockIdx.x, split = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int l16 = lane & 15, kg = lane >> 4;
  T* Vs = reinterpret_cast<T*>(smem) + wv * (DEC_TK * VS);

  const int k0 = p.cu_k[b], len = p.cu_k[b + 1] - k0;
  int n_keys, tpb;
  const int n_tiles = dec_tiles<MODE>(p, b, len, n_keys, tpb);
  const int t_lo = split * DEC_TPS;
  if (t_lo >= n_tiles) return;  // the merge kernel derives the number of live splits the same way
  const int t_hi = min(n_tiles, t_lo + DEC_TPS);
  const int32_t* sel = MODE == DEC_MODE_SELECTED ? p.topk_idx + ((int64_t)h * p.batch + b) * p.topk : nullptr;

  // B operand [k = d][n = column]: columns 0..g-1 = heads of the group, column g = scoring head (compressed mode)
  vec8 qreg[NS];
  {
    int hq_i = -1;
    if (l16 < p.g) hq_i = h * p.g + l16;
    else if (MODE == DEC_MODE_COMPRESSED && l16 == p.g) hq_i = p.score_head_as_written ? h : h * p.g;
    const T* qrow = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)max(hq_i, 0) * p.q_sh + 8 * kg;
#pragma unroll
    for (int s_ = 0; s_ < NS; ++s_) qreg[s_] = hq_i >= 0 ? load16<vec8>(qrow + 32 * s_) : zero8<T>();
  }
  const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)h * p.k_sh + 8 * kg;
  const T* vbase = reinterpret_cast<const T*>(p.v) + (int64_t)h * p.v_sh;
  const T* vtr = Vs + (4 * kg + (l16 >> 2)) * VS + 4 * (l16 & 3);

  float m = -INFINITY, l = 0.f;  // of column l16, replicated over the four key groups
  f32x4 oacc[NDT];               // O^T[d = 16 t + 4 kg + i][column l16]
#pragma unroll
  for (int t = 0; t < NDT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) oacc[t][i] = 0.f;

  for (int tt = t_lo + wv; tt < t_hi; tt += 4) {
    int row0, n_valid;
    if (MODE == DEC_MODE_COMPRESSED) {
      row0 = tt * DEC_TK;
      n_valid = min(DEC_TK, n_keys - row0);
    } else {
      const int t = tt / tpb, sub = tt - t * tpb;
      const int blk = sel[t];
      bool dup = false;
      for (int u = 0; u < t; ++u) dup |= sel[u] == blk;
      row0 = blk * p.block_size + sub * DEC_TK;
      n_valid = (blk < 0 || dup) ? 0 : min(min(DEC_TK, p.block_size - sub * DEC_TK), len - row0);
    }
    if (n_valid <= 0) continue;  // uniform per wave
    // V rows (coalesced, 16 B per lane) are requested first so that they travel while S is computed
    vec8 vst[VCH];
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int c = lane + 64 * j, row = c / (D / 8), cc = c % (D / 8);
      vst[j] = zero8<T>();  // rows past n_valid are zero so that 0 * garbage cannot appear
      if (row < n_valid) vst[j] = load16_stream<vec8>(vbase + (int64_t)(k0 + row0 + row) * p.v_sn + cc * 8);
    }
    // S^T[key][column] = K Q^T, K fragments straight from global memory
    f32x4 acc[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int key = a * 16 + l16;
      const T* krow = kbase + (int64_t)(k0 + row0 + key) * p.k_sn;
      vec8 kf[NS];
#pragma unroll
      for (int s_ = 0; s_ < NS; ++s_) kf[s_] = key < n_valid ? load16_stream<vec8>(krow + 32 * s_) : zero8<T>();
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[a][i] = 0.f;
#pragma unroll
      for (int s_ = 0; s_ < NS; ++s_) acc[a] = Elem<T>::mfma16(kf[s_], qreg[s_], acc[a]);
    }
    if (MODE == DEC_MODE_COMPRESSED && p.raw_score && l16 == p.g) {
      float* rs = p.raw_score + ((int64_t)h * p.batch + b) * p.raw_ld + row0;
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const int key0 = a * 16 + 4 * kg;
        if (row0 + key0 < p.raw_ld) *reinterpret_cast<f32x4*>(rs + key0) = acc[a];
      }
    }
    float mx = m;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = a * 16 + 4 * kg + i;
        const float sv = key < n_valid ? acc[a][i] : -INFINITY;
        acc[a][i] = sv;
        mx = fmaxf(mx, sv);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mref = mx * p.scale_log2;  // n_valid > 0, so mx is finite
    const float alpha = exp2f(m * p.scale_log2 - mref);
    float lsum = 0.f;
    vec8 pk;  // contraction index 8 kg + j  <->  key 4 kg + j (j < 4), 16 + 4 kg + j - 4 (j >= 4)
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = fast_exp2(acc[a][i] * p.scale_log2 - mref);
        lsum += pv;
        pk[a * 4 + i] = (T)pv;
      }
    lsum += __shfl_xor(lsum, 16, 64);
    lsum += __shfl_xor(lsum, 32, 64);
    l = l * alpha + lsum;
    m = mx;
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int c = lane + 64 * j, row = c / (D / 8), cc = c % (D / 8);
      store16(&Vs[row * VS + cc * 8], vst[j]);
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int t = 0; t < NDT; ++t) {
#pragma unroll
      for (int i = 0; i < 4; ++i) oacc[t][i] *= alpha;
      vec8 vf = lds_read_tr8<T>(vtr + 16 * t, 16 * VS);  // V^T[d = 16 t + l16][keys in the order of pk]
      oacc[t] = Elem<T>::mfma16(vf, pk, oacc[t]);
    }
    __builtin_amdgcn_wave_barrier();
  }

  // merge the four waves through LDS, then one fp32 partial per work-group
  __syncthreads();
  float* mg = reinterpret_cast<float*>(smem);
  constexpr int PER = D * 16 + 32;
  float* mine = mg + wv * PER;
  if (kg == 0) {
    mine[l16] = m * p.scale_log2;
    mine[16 + l16] = l;
  }
#pragma unroll
  for (int t = 0; t < NDT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) mine[32 + (16 * t + 4 * kg + i) * 16 + l16] = oacc[t][i];
  __syncthreads();
  float* out = p.part + (((int64_t)b * p.hkv + h) * p.nsplit + split) * (p.g * (2 + D));
  for (int e = tid; e < p.g * D; e += 256) {
    const int col = e / D, d = e - col * D;
    float mt = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) mt = fmaxf(mt, mg[w * PER + col]);
    float lt = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = mg[w * PER + col];
      const float wgt = mw == -INFINITY ? 0.f : exp2f(mw - mt);
      lt += wgt * mg[w * PER + 16 + col];
      o += wgt * mg[w * PER + 32 + d * 16 + col];
    }
    out[col * (2 + D) + 2 + d] = o;
    if (d == 0) {
      out[col * (2 + D)] = mt;
      out[col * (2 + D) + 1] = lt;
    }
  }
}

// partials of a request -> o, lse (fixed order over the splits)
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
decode_merge_kernel(DecParams p, int D) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int len = p.cu_k[b + 1] - p.cu_k[b];
  int n_keys, tpb;
  const int n_tiles = dec_tiles<MODE>(p, b, len, n_keys, tpb);
  const int ns = (n_tiles + DEC_TPS - 1) / DEC_TPS;
  const int slot = p.g * (2 + D);
  const float* part = p.part + ((int64_t)b * p.hkv + h) * p.nsplit * slot;
  for (int e = threadIdx.x; e < p.g * D; e += 256) {
    const int col = e / D, d = e - col * D;
    const float* pc = part + col * (2 + D);
    float mt = -INFINITY;
#pragma unroll 8
    for (int s_ = 0; s_ < ns; ++s_) mt = fmaxf(mt, pc[s_ * slot]);
    float lt = 0.f, o = 0.f;
    // batches of loads issued together; the sums keep the order of the splits
    constexpr int UB = 8;
    for (int sb = 0; sb < ns; sb += UB) {
      float ms[UB], ls[UB], os[UB];
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        const int s_ = min(sb + u, ns - 1);
        ms[u] = pc[s_ * slot];
        ls[u] = pc[s_ * slot + 1];
        os[u] = pc[s_ * slot + 2 + d];
      }
#pragma unroll
      for (int u = 0; u < UB; ++u)
        if (sb + u < ns) {
          const float wgt = ms[u] == -INFINITY ? 0.f : exp2f(ms[u] - mt);
          lt += wgt * ls[u];
          o += wgt * os[u];
        }
    }
    const float inv_l = lt > 0.f ? 1.f / lt : 0.f;
    const int hq_i = h * p.g + col;
    reinterpret_cast<T*>(p.o)[((int64_t)b * p.hq + hq_i) * D + d] = (T)(o * inv_l);
    if (d == 0) p.lse[(int64_t)hq_i * p.batch + b] = lt > 0.f ? mt + log2f(lt) : -INFINITY;
  }
}

// ------------------------------------------------------------------ top-k ----
struct DecTopkParams {
  const float* raw_score;  // [Hkv, B, raw_ld]
  int64_t raw_ld;
  const float* lse;        // [Hq, B]
  const int32_t* cu_ck;    // [B+1] compressed rows per request
  const int32_t* pos;      // [B]
  const int32_t* seqlens;  // [B] cache length including the new token
  int batch, hkv, g;
  int kernel_size, kernel_stride, block_size, topk, init_blocks, local_blocks;
  int as_written;
  float scale_log2;
  int32_t* topk_idx;       // [Hkv, B, topk]
  float* block_score;      // optional [Hkv, B, score_ld]
  int64_t score_ld;
};

// one work-group per (request, kv head): the block scores stay in LDS, every selection round is an arg-max
// over the work-group (value first, lower block id on equal values)
constexpr int DEC_TOPK_THREADS = 256;

__global__ void __launch_bounds__(DEC_TOPK_THREADS)
decode_topk_kernel(DecTopkParams p) {
  extern __shared__ float bs[];
  __shared__ float wbest[DEC_TOPK_THREADS / WAVE];
  __shared__ int wbest_id[DEC_TOPK_THREADS / WAVE];
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & (WAVE - 1), wv = tid / WAVE;
  const int nc = p.cu_ck[b + 1] - p.cu_ck[b];
  const int qp = p.pos[b];
  const int n_vis = qp >= p.kernel_size - 1 ? min(nc, (qp - p.kernel_size + 1) / p.kernel_stride + 1) : 0;
  const int len = p.seqlens[b];
  const int nblk = p.as_written ? (nc + p.block_size - 1) / p.block_size : (len + p.block_size - 1) / p.block_size;
  const int bq = p.as_written ? 0 : (len - 1) / p.block_size;
  const int hq_s = p.as_written ? h : h * p.g;
  const float lse_r = p.lse[(int64_t)hq_s * p.batch + b];
  const int na = p.kernel_size / p.kernel_stride, ne = p.block_size / p.kernel_stride;
  const int n_off = na + ne - 1, pad = na - 1;
  const float* rs = p.raw_score + ((int64_t)h * p.batch + b) * p.raw_ld;
  for (int blk = tid; blk < nblk; blk += DEC_TOPK_THREADS) {
    float acc = 0.f;
    const int c0 = blk * ne - pad;
    for (int o = 0; o < n_off; ++o) {
      const int c = c0 + o;
      if (c >= 0 && c < n_vis) {
        const int wgt = min(min(o, n_off - 1 - o), min(na, ne) - 1) + 1;
        acc += (float)wgt * fast_exp2(rs[c] * p.scale_log2 - lse_r);
      }
    }
    if (blk < p.init_blocks || (bq >= blk && bq < blk + p.local_blocks)) acc = INFINITY;
    bs[blk] = acc;
    if (p.block_score) p.block_score[((int64_t)h * p.batch + b) * p.score_ld + blk] = acc;
  }
  if (p.block_score)
    for (int64_t blk = nblk + tid; blk < p.score_ld; blk += DEC_TOPK_THREADS)
      p.block_score[((int64_t)h * p.batch + b) * p.score_ld + blk] = -INFINITY;
  __syncthreads();
  int32_t* out = p.topk_idx + ((int64_t)h * p.batch + b) * p.topk;
  for (int t = 0; t < p.topk; ++t) {
    float best = -2.f;
    int best_id = 0x7fffffff;
    for (int blk = tid; blk < nblk; blk += DEC_TOPK_THREADS) {  // ascending ids: the first maximum is kept
      const float vv = bs[blk];
      if (vv > best) {
        best = vv;
        best_id = blk;
      }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(best_id, o, 64);
      if (ov > best || (ov == best && oi < best_id)) {
        best = ov;
        best_id = oi;
      }
    }
    if (lane == 0) {
      wbest[wv] = best;
      wbest_id[wv] = best_id;
    }
    __syncthreads();
    best = wbest[0];
    best_id = wbest_id[0];
#pragma unroll
    for (int w = 1; w < DEC_TOPK_THREADS / WAVE; ++w) {
      const float ov = wbest[w];
      const int oi = wbest_id[w];
      if (ov > best || (ov == best && oi < best_id)) {
        best = ov;
        best_id = oi;
      }
    }
    if (tid == 0) {
      out[t] = best >= 0.f ? best_id : -1;  // fewer than topk blocks exist
      if (best >= 0.f) bs[best_id] = -1.f;
    }
    __syncthreads();
  }
}

template <typename T, int D, int MODE>
static int dec_launch(const DecParams& p, hipStream_t stream) {
  constexpr int lds = DecLds<D>::BYTES;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)decode_attn_kernel<T, D, MODE>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) {
      set_error("hipFuncSetAttribute(%d B LDS): %s", lds, hipGetErrorString(e));
      return (int)e;
    }
  }
  ProfScope ps_(MODE == DEC_MODE_COMPRESSED ? "decode_cmpattn" : "decode_selattn", stream);
  if (p.nsplit > 0) decode_attn_kernel<T, D, MODE><<<dim3(p.hkv, p.nsplit, p.batch), 256, lds, stream>>>(p);
  decode_merge_kernel<T, MODE><<<dim3(p.batch, p.hkv), 256, 0, stream>>>(p, D);
  return 0;
}

template <int MODE>
static int dec_dispatch(int dtype, int head_dim, const DecParams& p, hipStream_t stream) {
  if (dtype == FSA_BF16) {
    if (head_dim == 64) return dec_launch<__bf16, 64, MODE>(p, stream);
    if (head_dim == 128) return dec_launch<__bf16, 128, MODE>(p, stream);
    if (head_dim == 256) return dec_launch<__bf16, 256, MODE>(p, stream);
  } else {
    if (head_dim == 64) return dec_launch<_Float16, 64, MODE>(p, stream);
    if (head_dim == 128) return dec_launch<_Float16, 128, MODE>(p, stream);
    if (head_dim == 256) return dec_launch<_Float16, 256, MODE>(p, stream);
  }
  set_error("decode: head_dim=%d not supported (64, 128, 256)", head_dim);
  return FSA_ERR_UNSUPPORTED;
}

static int dec_splits(int64_t max_keys) {
  const int64_t tiles = (max_keys + DEC_TK - 1) / DEC_TK;
  return (int)((tiles + DEC_TPS - 1) / DEC_TPS);
}
static size_t dec_ws_bytes(int batch, int hq, int hkv, int d, int64_t max_keys) {
  return (size_t)batch * hkv * (size_t)(dec_splits(max_keys) > 0 ? dec_splits(max_keys) : 1) * (hq / hkv) * (2 + d) * 4;
}

}  // namespace fsa

using namespace fsa;

extern "C" size_t fsa_decode_workspace_bytes(int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                             int32_t head_dim, int64_t max_keys) {
  if (batch < 1 || num_kv_heads < 1 || num_q_heads % num_kv_heads || max_keys < 0) return 0;
  return dec_ws_bytes(batch, num_q_heads, num_kv_heads, head_dim, max_keys);
}

extern "C" int fsa_decode_cmpattn(const void* q, const void* ck, const void* cv, int32_t dtype,
                                  int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_n,
                                  int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                                  const int32_t* cu_ck, const int32_t* pos, int32_t batch,
                                  int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                  int32_t kernel_size, int32_t kernel_stride, float softmax_scale,
                                  int32_t score_head_as_written, int64_t max_keys, void* o, float* lse,
                                  float* raw_score, int64_t raw_ld, void* workspace, size_t workspace_bytes,
                                  void* stream_) {
  FSA_CHECK_ARG(q && ck && cv && cu_ck && pos && o && lse, "fsa_decode_cmpattn: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_decode_cmpattn: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(num_kv_heads >= 1 && num_q_heads % num_kv_heads == 0,
                "fsa_decode_cmpattn: num_q_heads must be a multiple of num_kv_heads");
  const int g = num_q_heads / num_kv_heads;
  FSA_CHECK_ARG(g <= 15, "fsa_decode_cmpattn: at most 15 query heads per kv head");
  FSA_CHECK_ARG(max_keys >= 0 && max_keys < (1ll << 30), "fsa_decode_cmpattn: bad max_keys");
  FSA_CHECK_ARG(workspace && workspace_bytes >= dec_ws_bytes(batch, num_q_heads, num_kv_heads, head_dim, max_keys),
                "fsa_decode_cmpattn: workspace too small (see fsa_decode_workspace_bytes)");
  FSA_CHECK_ARG(batch >= 1 && kernel_size >= 1 && kernel_stride >= 1, "fsa_decode_cmpattn: bad sizes");
  FSA_CHECK_ARG(!raw_score || (raw_ld >= 4 && raw_ld % 4 == 0), "fsa_decode_cmpattn: raw_ld must be a multiple of 4");
  FSA_CHECK_ARG(!score_head_as_written || num_kv_heads <= num_q_heads, "fsa_decode_cmpattn: bad scoring head");
  DecParams p = {};
  p.q = q; p.k = ck; p.v = cv; p.q_sb = q_stride_b; p.q_sh = q_stride_h;
  p.k_sn = k_stride_n; p.k_sh = k_stride_h; p.v_sn = v_stride_n; p.v_sh = v_stride_h;
  p.cu_k = cu_ck; p.pos = pos; p.batch = batch; p.hq = num_q_heads; p.hkv = num_kv_heads; p.g = g;
  p.kernel_size = kernel_size; p.kernel_stride = kernel_stride; p.scale_log2 = softmax_scale * LOG2E;
  p.o = o; p.lse = lse; p.raw_score = raw_score; p.raw_ld = raw_ld;
  p.score_head_as_written = score_head_as_written;
  p.part = (float*)workspace; p.nsplit = dec_splits(max_keys); p.max_keys = (int)max_keys;
  int rc = dec_dispatch<DEC_MODE_COMPRESSED>(dtype, head_dim, p, (hipStream_t)stream_);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_decode_cmpattn");
  return 0;
}

extern "C" int fsa_decode_topk(const float* raw_score, int64_t raw_ld, const float* lse,
                               const int32_t* cu_ck, const int32_t* pos, const int32_t* seqlens,
                               int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                               int32_t kernel_size, int32_t kernel_stride, int32_t block_size,
                               int32_t topk, int32_t init_blocks, int32_t local_blocks,
                               int32_t as_written, float softmax_scale, int64_t max_blocks,
                               int32_t* topk_idx, float* block_score, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(raw_score && lse && cu_ck && pos && seqlens && topk_idx, "fsa_decode_topk: null pointer");
  FSA_CHECK_ARG(batch >= 1 && topk >= 1 && num_kv_heads >= 1 && num_q_heads % num_kv_heads == 0,
                "fsa_decode_topk: bad sizes");
  FSA_CHECK_ARG(kernel_stride >= 1 && kernel_size % kernel_stride == 0 && block_size % kernel_stride == 0,
                "fsa_decode_topk: kernel_size and block_size must be multiples of kernel_stride");
  FSA_CHECK_ARG(max_blocks >= 1 && max_blocks * 4 <= 64 * 1024,
                "fsa_decode_topk: max_blocks must be in [1, 16384]");
  DecTopkParams p = {};
  p.raw_score = raw_score; p.raw_ld = raw_ld; p.lse = lse; p.cu_ck = cu_ck; p.pos = pos; p.seqlens = seqlens;
  p.batch = batch; p.hkv = num_kv_heads; p.g = num_q_heads / num_kv_heads;
  p.kernel_size = kernel_size; p.kernel_stride = kernel_stride; p.block_size = block_size; p.topk = topk;
  p.init_blocks = init_blocks; p.local_blocks = local_blocks; p.as_written = as_written;
  p.scale_log2 = softmax_scale * LOG2E; p.topk_idx = topk_idx; p.block_score = block_score;
  p.score_ld = max_blocks;
  {
    ProfScope ps_("decode_topk", stream);
    decode_topk_kernel<<<dim3(batch, num_kv_heads), DEC_TOPK_THREADS, (size_t)max_blocks * 4, stream>>>(p);
  }
  FSA_CHECK_LAUNCH("fsa_decode_topk");
  return 0;
}

extern "C" int fsa_decode_selattn(const void* q, const void* k_cache, const void* v_cache, int32_t dtype,
                                  int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_n,
                                  int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                                  const int32_t* cu_k, const int32_t* topk_idx, int32_t batch,
                                  int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                  int32_t topk, int32_t block_size, float softmax_scale, void* o,
                                  float* lse, void* workspace, size_t workspace_bytes, void* stream_) {
  FSA_CHECK_ARG(q && k_cache && v_cache && cu_k && topk_idx && o && lse, "fsa_decode_selattn: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_decode_selattn: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(num_kv_heads >= 1 && num_q_heads % num_kv_heads == 0,
                "fsa_decode_selattn: num_q_heads must be a multiple of num_kv_heads");
  FSA_CHECK_ARG(num_q_heads / num_kv_heads <= 16, "fsa_decode_selattn: at most 16 query heads per kv head");
  FSA_CHECK_ARG(batch >= 1 && topk >= 1 && block_size >= 1, "fsa_decode_selattn: bad sizes");
  const int64_t max_keys = (int64_t)topk * ((block_size + DEC_TK - 1) / DEC_TK) * DEC_TK;
  FSA_CHECK_ARG(workspace && workspace_bytes >= dec_ws_bytes(batch, num_q_heads, num_kv_heads, head_dim, max_keys),
                "fsa_decode_selattn: workspace too small (see fsa_decode_workspace_bytes)");
  DecParams p = {};
  p.q = q; p.k = k_cache; p.v = v_cache; p.q_sb = q_stride_b; p.q_sh = q_stride_h;
  p.k_sn = k_stride_n; p.k_sh = k_stride_h; p.v_sn = v_stride_n; p.v_sh = v_stride_h;
  p.cu_k = cu_k; p.topk_idx = topk_idx; p.batch = batch; p.hq = num_q_heads; p.hkv = num_kv_heads;
  p.g = num_q_heads / num_kv_heads; p.topk = topk; p.block_size = block_size;
  p.scale_log2 = softmax_scale * LOG2E; p.o = o; p.lse = lse;
  p.part = (float*)workspace; p.nsplit = dec_splits(max_keys);
  int rc = dec_dispatch<DEC_MODE_SELECTED>(dtype, head_dim, p, (hipStream_t)stream_);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_decode_selattn");
  return 0;
}
