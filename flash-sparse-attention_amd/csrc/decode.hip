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
// only).  The 32-key tiles of all (request, kv head) pairs form one sequence,
// and a persistent grid of single-wave work-groups - as many as are resident
// on the chip at once - cuts it into equal contiguous shares: no work-group is
// dispatched while the kernel runs, every wave streams for the whole launch
// and always has the rows of its next tile in flight while it computes the
// current one.  The rows of a tile arrive row-coalesced (16 B per lane, whole
// 2*D-byte rows per instruction) and pass through a wave-private LDS tile: K
// is read back as 16x16x32 MFMA operands, V transposed.  A wave writes one
// fp32 partial (m, l, O) per pair it touches; a small merge kernel combines
// the partials of a pair in a fixed order.  The query heads occupy the first
// g of the 16 MFMA columns; column g carries the scoring head.
//
// Semantics: fsa_preview/ops/compressed_attention_decode.py:361-490 (attention),
// :494-592 (scores), :284-357 (transform), :203-205 (top-k);
// fsa_preview/ops/selected_attention_decode.py:8-42.
#include "fsa_common.h"

#include <mutex>

namespace fsa {

constexpr int DEC_MODE_COMPRESSED = 0;
constexpr int DEC_MODE_SELECTED = 1;
constexpr int DEC_TK = 32;            // keys per wave tile
constexpr int DEC_MAX_WAVES = 4096;   // upper bound of the persistent grid (the workspace is sized for it)
// resident waves per SIMD the register budget is set for (head_dim 256 stages twice the rows per tile)
template <int D> struct DecOcc { static constexpr int WAVES_PER_SIMD = D >= 256 ? 1 : 2; };

struct DecParams {
  const void* q;   // [B, Hq, D]
  const void* k;   // [total, Hkv, D]
  const void* v;
  int64_t q_sb, q_sh, k_sn, k_sh, v_sn, v_sh;
  const int32_t* cu_k;      // [B+1] rows of k / v per request
  const int32_t* pos;       // compressed mode: position of the query
  const int32_t* topk_idx;  // selected mode: [Hkv, B, T]
  const int32_t* seqlens;   // selected mode, optional: [B] valid rows of each request's slot (null: the whole slot)
  int batch, hq, hkv, g, topk, block_size, kernel_size, kernel_stride;
  // One launch covers the heads [head0, head0 + g) of every GQA group of gq heads (the 16 columns of the MFMA tile
  // hold at most 16 heads): groups of more heads are served by several launches over the same workspace.
  int gq, head0;
  int score_col;            // compressed mode with raw_score: the column whose unscaled scores are kept
  float scale_log2;
  void* o;                  // [B, Hq, D] contiguous
  float* lse;               // [Hq, B]
  float* raw_score;         // compressed mode, optional: [Hkv, B, raw_ld] unscaled q.k of the scoring head
  int64_t raw_ld;
  int score_head_as_written;  // 0: first head of the group, 1: q-head with the kv head's own index
  int max_keys;             // compressed mode: host upper bound of the visible keys of a request (more are ignored)
  float* part;              // [slot][g][4 + D]: base-2 scaled max, sum, 2 unused, unnormalised O
  int32_t* tile_prefix;     // [B+1]: tiles (over all kv heads) of the requests before b
};

template <int D> struct DecLds {
  static constexpr int VS = D + 8;
  static constexpr int BYTES = DEC_TK * VS * 2;  // one wave's tile
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

// tile_prefix[b] = kv heads x tiles of the requests before b (one wave, scan over the requests)
template <int MODE>
__global__ void __launch_bounds__(WAVE)
decode_plan_kernel(DecParams p) {
  const int lane = threadIdx.x;
  int carry = 0;
  for (int b0 = 0; b0 < p.batch; b0 += WAVE) {
    const int b = b0 + lane;
    int nt = 0;
    if (b < p.batch) {
      int n_keys, tpb;
      nt = dec_tiles<MODE>(p, b, p.cu_k[b + 1] - p.cu_k[b], n_keys, tpb) * p.hkv;
    }
    int incl = nt;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
      const int y = __shfl_up(incl, o, WAVE);
      if (lane >= o) incl += y;
    }
    if (b < p.batch) p.tile_prefix[b] = carry + incl - nt;
    carry += __shfl(incl, WAVE - 1, WAVE);
  }
  if (lane == 0) p.tile_prefix[p.batch] = carry;
}

// Tiles before request b.  Selected mode: every request has topk x tiles-per-block tiles per kv head, so the
// prefix is a product and the plan kernel is not needed.
template <int MODE> __device__ __forceinline__ int dec_prefix(const DecParams& p, int b) {
  if (MODE == DEC_MODE_SELECTED) return b * (p.topk * ((p.block_size + DEC_TK - 1) / DEC_TK) * p.hkv);
  return p.tile_prefix[b];
}
// request that holds tile x of the sequence (x < total)
template <int MODE> __device__ __forceinline__ int dec_request_of(const DecParams& p, int x) {
  if (MODE == DEC_MODE_SELECTED) return x / (p.topk * ((p.block_size + DEC_TK - 1) / DEC_TK) * p.hkv);
  return upper_seg(p.tile_prefix, p.batch, x);
}

// share of the tile sequence per wave for a grid of n_waves
__device__ __forceinline__ int dec_share(int total, int n_waves) { return max(1, (total + n_waves - 1) / n_waves); }

template <typename T, int D, int MODE>
__global__ void __launch_bounds__(WAVE, DecOcc<D>::WAVES_PER_SIMD)
decode_attn_kernel(DecParams p) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int VS = DecLds<D>::VS;
  constexpr int NS = D / 32, NDT = D / 16, VCH = DEC_TK * (D / 8) / 64, PS = D + 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Vs = reinterpret_cast<T*>(smem);
  const int lane = threadIdx.x, l16 = lane & 15, kg = lane >> 4;
  const int w = blockIdx.x;
  const int total = dec_prefix<MODE>(p, p.batch);
  const int per = dec_share(total, gridDim.x);
  const int x_lo = w * per, x_hi = min(total, x_lo + per);
  if (x_lo >= x_hi) return;

  // position in the tile sequence: request (with its sizes), kv head, tile of the pair
  struct Req { int b, k0, len, n_keys, tpb, nt; };
  auto load_req = [&](Req& r, int b) {
    r.b = b;
    r.k0 = p.cu_k[b];
    r.len = p.cu_k[b + 1] - r.k0;
    if (MODE == DEC_MODE_SELECTED && p.seqlens) r.len = max(0, min(r.len, p.seqlens[b]));
    r.nt = dec_tiles<MODE>(p, b, r.len, r.n_keys, r.tpb);
  };
  // first cache row and number of valid keys (0: nothing to do) of a tile
  auto tile_desc = [&](const Req& r, int h, int tt, int& row0, int& n_valid) {
    if (MODE == DEC_MODE_COMPRESSED) {
      row0 = tt * DEC_TK;
      n_valid = min(DEC_TK, r.n_keys - row0);
    } else {
      const int32_t* sel = p.topk_idx + ((int64_t)h * p.batch + r.b) * p.topk;
      const int t = tt / r.tpb, sub = tt - t * r.tpb;
      const int blk = sel[t];
      bool dup = false;
      for (int u = 0; u < t; ++u) dup |= sel[u] == blk;
      row0 = blk * p.block_size + sub * DEC_TK;
      n_valid = (blk < 0 || dup) ? 0 : min(min(DEC_TK, p.block_size - sub * DEC_TK), r.len - row0);
    }
    n_valid = max(n_valid, 0);
    row0 = n_valid > 0 ? row0 : 0;
  };
  // rows of a tile, coalesced (16 B per lane, D/8 lanes per row); rows past n_valid are zero so that
  // 0 * garbage cannot appear
  // (the offsets inside a tile fit 32 bits: uniform base pointer + one offset register per lane)
  auto load_tile = [&](vec8 (&dst)[VCH], const T* base, int64_t sn, int n_valid) {
    constexpr int RPI = 64 / (D / 8);  // rows per load instruction
    const uint32_t off0 = (uint32_t)(lane / (D / 8)) * (uint32_t)sn + (uint32_t)(lane % (D / 8)) * 8u;
    const uint32_t step = (uint32_t)RPI * (uint32_t)sn;
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int row = lane / (D / 8) + RPI * j;
      dst[j] = zero8<T>();
      if (row < n_valid) dst[j] = load16_stream<vec8>(base + (off0 + step * (uint32_t)j));
    }
  };
  auto park_tile = [&](const vec8 (&src)[VCH]) {
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int c = lane + 64 * j, row = c / (D / 8), cc = c % (D / 8);
      store16(&Vs[row * VS + cc * 8], src[j]);
    }
  };
  // B operand [k = d][n = column]: columns 0..g-1 = heads of the group, column g = scoring head (compressed mode)
  vec8 qreg[NS];
  auto load_q = [&](int b, int h) {
    int hq_i = -1;
    if (l16 < p.g) hq_i = h * p.gq + p.head0 + l16;
    else if (MODE == DEC_MODE_COMPRESSED && p.raw_score && l16 == p.score_col) hq_i = h;  // as written: head h of q
    const T* qrow = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)max(hq_i, 0) * p.q_sh + 8 * kg;
#pragma unroll
    for (int s_ = 0; s_ < NS; ++s_) qreg[s_] = hq_i >= 0 ? load16<vec8>(qrow + 32 * s_) : zero8<T>();
  };
  const T* kall = reinterpret_cast<const T*>(p.k);
  const T* vall = reinterpret_cast<const T*>(p.v);
  const T* vtr = Vs + (4 * kg + (l16 >> 2)) * VS + 4 * (l16 & 3);

  float m = -INFINITY, l = 0.f;  // of column l16, replicated over the four key groups
  f32x4 oacc[NDT];               // O^T[d = 16 t + 4 kg + i][column l16]
#pragma unroll
  for (int t = 0; t < NDT; ++t) oacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  Req rq, rqn;
  load_req(rq, dec_request_of<MODE>(p, x_lo));
  int h, tt;
  {
    const int rem = x_lo - dec_prefix<MODE>(p, rq.b);
    h = rem / rq.nt;
    tt = rem - h * rq.nt;
  }
  rqn = rq;
  int hn = h, ttn = tt;
  int row0, n_valid;
  tile_desc(rq, h, tt, row0, n_valid);
  vec8 kst[VCH], vst[VCH];
  load_tile(kst, kall + (int64_t)(rq.k0 + row0) * p.k_sn + (int64_t)h * p.k_sh, p.k_sn, n_valid);
  load_tile(vst, vall + (int64_t)(rq.k0 + row0) * p.v_sn + (int64_t)h * p.v_sh, p.v_sn, n_valid);
  load_q(rq.b, h);

  for (int x = x_lo; x < x_hi; ++x) {
    const bool has_next = x + 1 < x_hi;
    int row0n = 0, n_validn = 0;
    if (has_next) {  // x + 1 < total: a further tile exists
      if (++ttn == rqn.nt) {
        ttn = 0;
        if (++hn == p.hkv) {
          hn = 0;
          do load_req(rqn, rqn.b + 1); while (rqn.nt == 0);
        }
      }
      tile_desc(rqn, hn, ttn, row0n, n_validn);
    }
    const bool live = n_valid > 0;  // uniform
    // the K rows go through the LDS tile first, V uses it afterwards; the rows of the next tile are requested as
    // soon as the staging registers are free, so that they travel while this tile is computed
    if (live) park_tile(kst);
    load_tile(kst, kall + (int64_t)(rqn.k0 + row0n) * p.k_sn + (int64_t)hn * p.k_sh, p.k_sn, n_validn);
    float alpha = 1.f;
    vec8 pk = zero8<T>();  // contraction index 8 kg + j  <->  key 4 kg + j (j < 4), 16 + 4 kg + j - 4 (j >= 4)
    if (live) {
      __builtin_amdgcn_wave_barrier();
      // S^T[key][column] = K Q^T
      f32x4 acc[2];
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        acc[a] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s_ = 0; s_ < NS; ++s_) {
          vec8 kf = load16<vec8>(&Vs[(a * 16 + l16) * VS + 32 * s_ + 8 * kg]);
          acc[a] = Elem<T>::mfma16(kf, qreg[s_], acc[a]);
        }
      }
      __builtin_amdgcn_wave_barrier();
      if (MODE == DEC_MODE_COMPRESSED && p.raw_score && l16 == p.score_col) {
        float* rs = p.raw_score + ((int64_t)h * p.batch + rq.b) * p.raw_ld + row0;
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
      alpha = exp2f(m * p.scale_log2 - mref);
      float lsum = 0.f;
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
      park_tile(vst);
    }
    load_tile(vst, vall + (int64_t)(rqn.k0 + row0n) * p.v_sn + (int64_t)hn * p.v_sh, p.v_sn, n_validn);
    if (live) {
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
    if (!has_next || hn != h || rqn.b != rq.b) {
      // last tile of the pair in this wave's share: the partial of (wave, pair) goes to slot wave + pair, which
      // no other (wave, pair) can name because the shares are contiguous
      float* out = p.part + (int64_t)(w + rq.b * p.hkv + h) * (p.g * PS);
      if (l16 < p.g) {
        float* oc = out + l16 * PS;
        if (kg == 0) *reinterpret_cast<f32x4*>(oc) = f32x4{m * p.scale_log2, l, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < NDT; ++t) *reinterpret_cast<f32x4*>(oc + 4 + 16 * t + 4 * kg) = oacc[t];
      }
      m = -INFINITY;
      l = 0.f;
#pragma unroll
      for (int t = 0; t < NDT; ++t) oacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (has_next) load_q(rqn.b, hn);
    }
    rq = rqn;
    h = hn;
    tt = ttn;
    row0 = row0n;
    n_valid = n_validn;
  }
}

// partials of a pair -> o, lse (fixed order over the waves that shared its tiles)
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
decode_merge_kernel(DecParams p, int D, int n_waves) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int len = p.cu_k[b + 1] - p.cu_k[b];
  int n_keys, tpb;
  const int nt = dec_tiles<MODE>(p, b, len, n_keys, tpb);
  const int per = dec_share(dec_prefix<MODE>(p, p.batch), n_waves);
  const int x0 = dec_prefix<MODE>(p, b) + h * nt;
  const int w0 = x0 / per;
  const int ns = nt > 0 ? (x0 + nt - 1) / per - w0 + 1 : 0;
  const int PS = D + 4, slot = p.g * PS;
  const float* part = p.part + (int64_t)(w0 + b * p.hkv + h) * slot;
  for (int e = threadIdx.x; e < p.g * D; e += 256) {
    const int col = e / D, d = e - col * D;
    const float* pc = part + col * PS;
    float mt = -INFINITY;
#pragma unroll 8
    for (int s_ = 0; s_ < ns; ++s_) mt = fmaxf(mt, pc[s_ * slot]);
    float lt = 0.f, o = 0.f;
    // batches of loads issued together; the sums keep the order of the waves
    constexpr int UB = 8;
    for (int sb = 0; sb < ns; sb += UB) {
      float ms[UB], ls[UB], os[UB];
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        const int s_ = min(sb + u, ns - 1);
        ms[u] = pc[s_ * slot];
        ls[u] = pc[s_ * slot + 1];
        os[u] = pc[s_ * slot + 4 + d];
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
    const int hq_i = h * p.gq + p.head0 + col;
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
  int scores_to_bf16;      // rank the block scores after rounding them to bf16 (what the prefill selection does)
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
    bs[blk] = p.scores_to_bf16 ? (float)(__bf16)acc : acc;
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
    {
      // scores are >= 0 (negative: nothing left in this lane): as 64-bit keys, score bits above and the complement of
      // the id below, the larger key is the larger score or, on equal scores, the lower id
      const uint64_t mine = best < 0.f ? 0ull : ((uint64_t)__float_as_uint(best) << 32) | (0xFFFFFFFFu - (uint32_t)best_id);
      const uint64_t top = wave_max_u64(mine);
      best = top ? __uint_as_float((uint32_t)(top >> 32)) : -2.f;
      best_id = top ? (int)(0xFFFFFFFFu - (uint32_t)top) : 0x7fffffff;
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

// number of single-wave work-groups that are resident at once on the current device
template <typename T, int D, int MODE>
static int dec_grid_waves(int* n_waves) {
  static int cached[16] = {0};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess && dev >= 0 && dev < 16 && cached[dev] > 0) {
    *n_waves = cached[dev];
    return 0;
  }
  int cus = 0, per_cu = 0;
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess)
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, decode_attn_kernel<T, D, MODE>, WAVE, DecLds<D>::BYTES);
  if (e != hipSuccess || cus < 1 || per_cu < 1) {
    set_error("decode: occupancy query failed (%s, %d CUs, %d work-groups per CU)", hipGetErrorString(e), cus, per_cu);
    return e != hipSuccess ? (int)e : FSA_ERR_UNSUPPORTED;
  }
  int n = cus * per_cu;
  if (n > DEC_MAX_WAVES) n = DEC_MAX_WAVES;
  if (dev >= 0 && dev < 16) cached[dev] = n;
  *n_waves = n;
  return 0;
}

// p0.g holds the whole group size on entry.  Scores of the scoring head: with the first head of the group as
// scoring head they are the scores of column 0 of the first launch; with the head that the reference's kernel
// actually reads (q head number h for kv head h) they need a column of their own, so that launch has 15 heads.
template <typename T, int D, int MODE>
static int dec_launch(const DecParams& p0, hipStream_t stream) {
  int n_waves = 0;
  int rc = dec_grid_waves<T, D, MODE>(&n_waves);
  if (rc) return rc;
  ProfScope ps_(MODE == DEC_MODE_COMPRESSED ? "decode_cmpattn" : "decode_selattn", stream);
  DecParams p = p0;
  p.gq = p0.g;
  if (MODE == DEC_MODE_COMPRESSED) decode_plan_kernel<MODE><<<1, WAVE, 0, stream>>>(p);
  for (int head0 = 0; head0 < p0.g;) {
    p.head0 = head0;
    p.raw_score = head0 == 0 ? p0.raw_score : nullptr;
    const bool own_col = MODE == DEC_MODE_COMPRESSED && p.raw_score && p0.score_head_as_written;
    p.g = std::min(p0.g - head0, own_col ? 15 : 16);
    p.score_col = own_col ? p.g : 0;
    decode_attn_kernel<T, D, MODE><<<n_waves, WAVE, DecLds<D>::BYTES, stream>>>(p);
    decode_merge_kernel<T, MODE><<<dim3(p.batch, p.hkv), 256, 0, stream>>>(p, D, n_waves);
    head0 += p.g;
  }
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

// workspace: tile prefix of the requests, then one partial slot per (wave, pair) that can occur
static size_t dec_ws_prefix_bytes(int batch) { return align_up((size_t)(batch + 1) * 4, 256); }
static size_t dec_ws_bytes(int batch, int hq, int hkv, int d) {
  return dec_ws_prefix_bytes(batch) + ((size_t)DEC_MAX_WAVES + (size_t)batch * hkv) * (hq / hkv) * (4 + d) * 4;
}

// Scratch memory of fsa_decode_selattn_static: lives in the code object, one copy per device that loads it, for
// as long as the process runs.  In host code the array's name is only a handle for hipGetSymbolAddress.
constexpr size_t DEC_STATIC_SCRATCH_BYTES = (size_t)FSA_DECODE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char dec_static_scratch[DEC_STATIC_SCRATCH_BYTES];

// Per-device state of the scratch array: its device address (looked up once), and the stream and completion
// event of the last call that used it.
struct DecStaticState {
  void* ptr = nullptr;
  hipEvent_t done = nullptr;
  hipStream_t last_stream = nullptr;
  bool used = false;
};
constexpr int DEC_STATIC_MAX_DEV = 64;
static DecStaticState dec_static_state[DEC_STATIC_MAX_DEV];
static std::mutex dec_static_mu;

// Set-up for one call on `stream`: the scratch address of the current device, and - the array is shared by every
// call on the device - an ordering edge behind the previous call when that one ran on another stream
// (hipStreamWaitEvent on its completion event; nothing is allocated per call, the event is created once per
// device).  Calls recorded into a graph take no part in this: a capturing stream may neither wait for nor record
// an event of eager work, so captured calls are ordered by the graph's own dependencies.
static int dec_static_begin(hipStream_t stream, void** out, bool* capturing) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("fsa_decode_selattn_static: hipGetDevice: %s", hipGetErrorString(e));
    return (int)e;
  }
  if (dev < 0 || dev >= DEC_STATIC_MAX_DEV) {
    set_error("fsa_decode_selattn_static: device %d out of range", dev);
    return FSA_ERR_UNSUPPORTED;
  }
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cs) != hipSuccess) {
    (void)hipGetLastError();
    cs = hipStreamCaptureStatusNone;
  }
  *capturing = cs != hipStreamCaptureStatusNone;
  std::lock_guard<std::mutex> lock(dec_static_mu);
  DecStaticState& st = dec_static_state[dev];
  if (!st.ptr) {
    void* a = nullptr;
    e = hipGetSymbolAddress(&a, HIP_SYMBOL(dec_static_scratch));
    if (e != hipSuccess || !a) {
      set_error("fsa_decode_selattn_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return e != hipSuccess ? (int)e : FSA_ERR_UNSUPPORTED;
    }
    st.ptr = a;
  }
  *out = st.ptr;
  if (*capturing) return 0;
  if (!st.done) {
    e = hipEventCreateWithFlags(&st.done, hipEventDisableTiming);
    if (e != hipSuccess) {
      set_error("fsa_decode_selattn_static: hipEventCreateWithFlags: %s", hipGetErrorString(e));
      return (int)e;
    }
  }
  if (st.used && st.last_stream != stream) {
    e = hipStreamWaitEvent(stream, st.done, 0);
    if (e != hipSuccess) {
      set_error("fsa_decode_selattn_static: hipStreamWaitEvent: %s", hipGetErrorString(e));
      return (int)e;
    }
  }
  return 0;
}

// After the kernels of an eager call are enqueued: remember its stream and mark its end.
static int dec_static_end(hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= DEC_STATIC_MAX_DEV) return 0;
  std::lock_guard<std::mutex> lock(dec_static_mu);
  DecStaticState& st = dec_static_state[dev];
  if (!st.done) return 0;
  hipError_t e = hipEventRecord(st.done, stream);
  if (e != hipSuccess) {
    set_error("fsa_decode_selattn_static: hipEventRecord: %s", hipGetErrorString(e));
    return (int)e;
  }
  st.last_stream = stream;
  st.used = true;
  return 0;
}

}  // namespace fsa

using namespace fsa;

extern "C" size_t fsa_decode_workspace_bytes(int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                             int32_t head_dim, int64_t max_keys) {
  if (batch < 1 || num_kv_heads < 1 || num_q_heads % num_kv_heads || max_keys < 0) return 0;
  return dec_ws_bytes(batch, num_q_heads, num_kv_heads, head_dim);
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
  FSA_CHECK_ARG(max_keys >= 0 && max_keys < (1ll << 30), "fsa_decode_cmpattn: bad max_keys");
  FSA_CHECK_ARG(workspace && workspace_bytes >= dec_ws_bytes(batch, num_q_heads, num_kv_heads, head_dim),
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
  p.tile_prefix = (int32_t*)workspace; p.part = (float*)((char*)workspace + dec_ws_prefix_bytes(batch));
  p.max_keys = (int)max_keys;
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
                               int32_t as_written, int32_t scores_to_bf16, float softmax_scale,
                               int64_t max_blocks, int32_t* topk_idx, float* block_score, void* stream_) {
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
  p.scores_to_bf16 = scores_to_bf16;
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
                                  const int32_t* cu_k, const int32_t* seqlens, const int32_t* topk_idx,
                                  int32_t batch, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                  int32_t topk, int32_t block_size, float softmax_scale, void* o,
                                  float* lse, void* workspace, size_t workspace_bytes, void* stream_) {
  FSA_CHECK_ARG(q && k_cache && v_cache && cu_k && topk_idx && o && lse, "fsa_decode_selattn: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_decode_selattn: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(num_kv_heads >= 1 && num_q_heads % num_kv_heads == 0,
                "fsa_decode_selattn: num_q_heads must be a multiple of num_kv_heads");
  FSA_CHECK_ARG(batch >= 1 && topk >= 1 && block_size >= 1, "fsa_decode_selattn: bad sizes");
  FSA_CHECK_ARG(workspace && workspace_bytes >= dec_ws_bytes(batch, num_q_heads, num_kv_heads, head_dim),
                "fsa_decode_selattn: workspace too small (see fsa_decode_workspace_bytes)");
  DecParams p = {};
  p.q = q; p.k = k_cache; p.v = v_cache; p.q_sb = q_stride_b; p.q_sh = q_stride_h;
  p.k_sn = k_stride_n; p.k_sh = k_stride_h; p.v_sn = v_stride_n; p.v_sh = v_stride_h;
  p.cu_k = cu_k; p.seqlens = seqlens; p.topk_idx = topk_idx; p.batch = batch; p.hq = num_q_heads;
  p.hkv = num_kv_heads; p.g = num_q_heads / num_kv_heads; p.topk = topk; p.block_size = block_size;
  p.scale_log2 = softmax_scale * LOG2E; p.o = o; p.lse = lse;
  p.tile_prefix = (int32_t*)workspace; p.part = (float*)((char*)workspace + dec_ws_prefix_bytes(batch));
  int rc = dec_dispatch<DEC_MODE_SELECTED>(dtype, head_dim, p, (hipStream_t)stream_);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_decode_selattn");
  return 0;
}

extern "C" int fsa_decode_selattn_static(const void* q, const void* k_cache, const void* v_cache, int32_t dtype,
                                         int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_n,
                                         int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                                         const int32_t* cu_k, const int32_t* seqlens, const int32_t* topk_idx,
                                         int32_t batch, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                         int32_t topk, int32_t block_size, float softmax_scale, void* o,
                                         float* lse, void* stream_) {
  FSA_CHECK_ARG(batch >= 1 && num_kv_heads >= 1 && num_q_heads >= 1 && num_q_heads % num_kv_heads == 0 &&
                    head_dim >= 1,
                "fsa_decode_selattn_static: bad sizes");
  const size_t need = dec_ws_bytes(batch, num_q_heads, num_kv_heads, head_dim);
  if (need > DEC_STATIC_SCRATCH_BYTES) {
    set_error("fsa_decode_selattn_static: batch %d x %d kv heads x %d heads per group x head_dim %d needs %zu bytes "
              "of scratch, the built-in buffer holds %zu; use fsa_decode_selattn with a caller workspace",
              batch, num_kv_heads, num_q_heads / num_kv_heads, head_dim, need, DEC_STATIC_SCRATCH_BYTES);
    return FSA_ERR_WORKSPACE;
  }
  void* scratch = nullptr;
  bool capturing = false;
  int rc = dec_static_begin((hipStream_t)stream_, &scratch, &capturing);
  if (rc) return rc;
  // every partial slot that the merge reads is written by the attention kernel of the same call: nothing in the
  // buffer has to start at zero
  rc = fsa_decode_selattn(q, k_cache, v_cache, dtype, q_stride_b, q_stride_h, k_stride_n, k_stride_h, v_stride_n,
                          v_stride_h, cu_k, seqlens, topk_idx, batch, num_q_heads, num_kv_heads, head_dim, topk, block_size,
                          softmax_scale, o, lse, scratch, DEC_STATIC_SCRATCH_BYTES, stream_);
  if (rc || capturing) return rc;
  return dec_static_end((hipStream_t)stream_);
}
