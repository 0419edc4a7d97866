// Selected attention forward for gfx950.
//
// Stage 1 (selattn_fwd_main_kernel): KV blocks on the outside.  A work-group
// owns one kv block of one kv head (K and V^T staged in LDS once) and a range
// of the gathered rows of that block; a row is one (query, head-in-group) pair,
// so a GQA group of any size fills MFMA tiles without padding.  Each wave takes
// 32 rows: S^T = K Q^T (32x32x16 MFMA, one row per lane), a single-block
// softmax in registers, O^T = V^T P^T, and writes the normalised partial row
// and its base-2 LSE.
// Stage 2 (selattn_fwd_reduce_kernel): query-major merge of the <= T partials
// of each (query, head) with shuffles, 16-byte coalesced loads, no atomics.
//
// Semantics follow fsa/ops/FSA_topk_sparse_attention.py:382-566 (main),
// :138-281 (reduce); the causal mask is q_pos >= key_pos (:520) and the LSE is
// base 2 (:256-261).
#include "fsa_common.h"

namespace fsa {

struct SelFwdParams {
  const void* q;
  const void* k;
  const void* v;
  int64_t q_sn, q_sh, k_sn, k_sh, v_sn, v_sh;
  const int32_t* cu_seqlens;
  const int32_t* cu_blocks;
  const int32_t* counts;
  const int32_t* starts;
  const int32_t* sel_tokens;
  const int32_t* tile_prefix;
  const int32_t* tile_block;  // [Hkv, max_tiles]: block of every tile
  int64_t max_tiles;
  int batch;
  int64_t max_blocks;
  int64_t cap;  // N * T: capacity of the per-head pair list
  int g;
  int g_shift;  // log2 g, or -1 if g is not a power of two
  float scale_log2;
  void* o_part;
  float* lse_part;
};

// Upper bound of the rows one work-group takes from a block (a block with more rows is dealt in equal shares to
// several work-groups): measured optimum about 3072 / 4096 / 6144-8192 rows for GQA groups of 1 / 2 / 4.
// Where LDS holds a single work-group per CU (head_dim 256, or 128-key blocks at head_dim 128) 1024 rows balance
// best.
static inline int sel_tile_rows(int g, int d, int bk) {
  const int kv_bytes = (bk * (d + 8) + bk * (d + 16)) * 2, stage_bytes = 32 * (d + 8) * 2;
  if (kv_bytes + 4 * stage_bytes > 80 * 1024) return 1024;   // SelLds<D, BK>::TWO_WGS is false
  const int r = 2048 + 1024 * g;
  return r < 8192 ? r : 8192;
}

template <int D, int BK> struct SelLds {
  static constexpr int KS = D + 8;   // K row stride in elements (16 B pad: bank spread)
  static constexpr int VS = D + 16;  // V row stride in elements (32 B pad for the transposing reads)
  static constexpr int OS = D + 8;   // row stride of the per-wave output staging tile
  static constexpr int KV_BYTES = (BK * KS + BK * VS) * 2;
  static constexpr int STAGE_BYTES = 32 * OS * 2;  // one wave's [32][D] tile
  // Four waves with staging tiles, two work-groups per CU, where that fits in LDS.  Otherwise one work-group
  // per CU: eight waves (two per SIMD) share the K / V copy, with staging tiles if LDS still holds them.
  static constexpr bool TWO_WGS = KV_BYTES + 4 * STAGE_BYTES <= 80 * 1024;
  static constexpr bool STAGE8 = KV_BYTES + 8 * STAGE_BYTES <= 160 * 1024;
  static constexpr bool STAGE4 = KV_BYTES + 4 * STAGE_BYTES <= 160 * 1024;
  static constexpr int THREADS = TWO_WGS ? 256 : (STAGE8 || !STAGE4) ? 512 : 256;
  static constexpr int NWAVES = THREADS / 64;
  static constexpr bool STAGE_OUT = KV_BYTES + NWAVES * STAGE_BYTES <= 160 * 1024;
  // where LDS cannot hold whole-row tiles: a [32][32] slice tile per wave, so that partial rows still leave in
  // 64-byte pieces, and Q fragments straight from global memory
  static constexpr int SLS = 32 + 8;
  static constexpr bool SLICE_OUT = !STAGE_OUT && KV_BYTES + NWAVES * 32 * SLS * 2 <= 160 * 1024;
  static constexpr int BYTES = KV_BYTES + (STAGE_OUT ? NWAVES * STAGE_BYTES : SLICE_OUT ? NWAVES * 32 * SLS * 2 : 0);
  static constexpr int WG_ROWS = NWAVES * 32;     // rows per pass of the work-group
  static constexpr int MIN_WAVES = (THREADS == 256 && D <= 128 && BK <= 64) ? 2 : 1;  // waves per SIMD the register budget allows
};

template <typename T, int D, int BK>
__global__ void __launch_bounds__((SelLds<D, BK>::THREADS), (SelLds<D, BK>::MIN_WAVES))
selattn_fwd_main_kernel(SelFwdParams p) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int KS = SelLds<D, BK>::KS, VS = SelLds<D, BK>::VS;
  constexpr int SEL_THREADS = SelLds<D, BK>::THREADS, SEL_WG_ROWS = SelLds<D, BK>::WG_ROWS;
  constexpr int NA = BK / 32;   // S^T accumulators (32 keys each)
  constexpr int NKS = D / 16;   // k-steps of QK^T
  constexpr int NDT = D / 32;   // O^T accumulators (32 dims each)
  constexpr int NJ = BK / 16;   // k-steps of PV
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Ks = reinterpret_cast<T*>(smem);
  T* Vs = Ks + BK * KS;
  constexpr int OS = SelLds<D, BK>::OS;
  T* Ost = Vs + BK * VS + (threadIdx.x >> 6) * (32 * OS);  // this wave's [32][D] staging tile
  constexpr int SLS = SelLds<D, BK>::SLS;
  T* Osl = Vs + BK * VS + (threadIdx.x >> 6) * (32 * SLS);  // or its [32][32] slice tile

  const int h = blockIdx.y;
  const int64_t nbp1 = p.max_blocks + 1;
  const int32_t* tp = p.tile_prefix + h * nbp1;
  const int w = blockIdx.x;
  if (w >= tp[p.max_blocks]) return;
  const int gb = p.tile_block[h * p.max_tiles + w];
  const int s = upper_seg(p.cu_blocks, p.batch, gb);
  const int b_local = gb - p.cu_blocks[s];
  const int seq_start = p.cu_seqlens[s], seq_end = p.cu_seqlens[s + 1];
  const int tok0 = seq_start + b_local * BK;
  const int rows = p.counts[h * p.max_blocks + gb] * p.g;
  const int start = p.starts[h * nbp1 + gb];
  // equal shares of the block's rows (whole passes) for its work-groups
  const int ntile_b = tp[gb + 1] - tp[gb];
  const int share = ((rows + ntile_b - 1) / ntile_b + SEL_WG_ROWS - 1) / SEL_WG_ROWS * SEL_WG_ROWS;
  const int row_lo = (w - tp[gb]) * share;
  const int row_hi = min(rows, row_lo + share);

  const int tid = threadIdx.x;
  const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)h * p.k_sh;
  const T* vbase = reinterpret_cast<const T*>(p.v) + (int64_t)h * p.v_sh;
  for (int c = tid; c < BK * (D / 8); c += SEL_THREADS) {
    const int row = c / (D / 8), col = c % (D / 8);
    const int tok = tok0 + row;
    vec8 x = zero8<T>();
    if (tok < seq_end) x = load16<vec8>(kbase + (int64_t)tok * p.k_sn + col * 8);
    store16(&Ks[row * KS + col * 8], x);
  }
  for (int c = tid; c < BK * (D / 8); c += SEL_THREADS) {
    const int row = c / (D / 8), col = c % (D / 8);
    const int tok = tok0 + row;
    vec8 x = zero8<T>();
    if (tok < seq_end) x = load16<vec8>(vbase + (int64_t)tok * p.v_sn + col * 8);
    store16(&Vs[row * VS + col * 8], x);
  }
  __syncthreads();

  const int lane = tid & 63, wv = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int32_t* toks = p.sel_tokens + (int64_t)h * p.cap + start;
  const T* qbase_row = reinterpret_cast<const T*>(p.q) + (int64_t)h * p.g * p.q_sh;
  const int64_t prow0 = ((int64_t)h * p.cap + start) * p.g;
  T* opart = reinterpret_cast<T*>(p.o_part);
  // this lane's address inside V for the transposing reads of O^T = V^T P^T:
  // keys 4*hh + (lane%16)/4 (+ 16*j, + 8), dims 16*((lane/16)&1) + 4*(lane%4) (+ 32*dt)
  const T* vtr = Vs + (4 * hh + ((lane & 15) >> 2)) * VS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  // Pipeline over the wave's 32-row sub-tiles.  Q rows are fetched with row-coalesced
  // 16-byte loads (CPR lanes cover one row, so a load instruction touches 8 cache lines
  // instead of 64) one sub-tile ahead, parked in registers, and pass through the wave's
  // LDS tile to reach the MFMA operand layout; token ids are fetched two steps ahead.
  constexpr int CPR = D / 8;      // 16-byte chunks per row
  constexpr int RPI = 64 / CPR;   // rows per load / store instruction
  constexpr int NLD = 32 / RPI;   // instructions per 32-row tile
  const int srow = lane / CPR, schunk = lane % CPR;
  const uint32_t q_sn32 = (uint32_t)p.q_sn, q_sh32 = (uint32_t)p.q_sh;
  auto row_token = [&](int sub_) {  // token id of row (sub_ + col), kept by lane col
    const int r_ = min(sub_ + col, row_hi - 1);
    return toks[div_group(r_, p.g, p.g_shift)];
  };
  auto fetch_q = [&](vec8 (&dst)[NLD], int tok_lane, int sub_) {
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
      const int row = srow + RPI * j;
      const int tok_ = __shfl(tok_lane, row, 64);
      const int r_ = min(sub_ + row, row_hi - 1);
      // strides and the head term fit 32 bits (checked by the host): one 32 x 32 -> 64 bit multiply-add per row
      const uint32_t head_ = p.g_shift >= 0 ? (uint32_t)(r_ & (p.g - 1)) : (uint32_t)(r_ - div_group(r_, p.g, p.g_shift) * p.g);
      dst[j] = load16<vec8>(qbase_row + ((uint64_t)(uint32_t)tok_ * q_sn32 + (head_ * q_sh32 + schunk * 8)));
    }
  };
  constexpr bool STAGED = SelLds<D, BK>::STAGE_OUT;  // false: LDS cannot hold the wave tiles, direct loads / stores
  vec8 qst[NLD], qst_b[NLD];   // staged mode: the rows of the next two sub-tiles wait here (two buffers in turn)
  // Direct mode: the Q fragments of a lane's row in the MFMA operand layout, straight from global memory.  k-step ks
  // contracts dims [16 ks, 16 ks + 16): the two lanes of a row read 32 contiguous bytes and a cache line is used up
  // by four consecutive loads.  Like qst they are requested one sub-tile ahead: as soon as the S^T products have
  // consumed them, while the softmax and the O^T products of the current sub-tile run.
  vec8 qdir[STAGED ? 1 : NKS];
  auto fetch_dir = [&](int token, int sub_) {
    const int rc_ = min(sub_ + col, row_hi - 1);
    const uint32_t head_ = (uint32_t)(rc_ - div_group(rc_, p.g, p.g_shift) * p.g);
    const T* qrow = qbase_row + ((uint64_t)(uint32_t)token * q_sn32 + (head_ * q_sh32 + hh * 8));
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) qdir[STAGED ? 0 : ks] = load16<vec8>(qrow + ks * 16);
  };
  // one sub-tile: rows sub.. of the block (direct mode: tok_next = token ids of the next sub-tile)
  // staged mode: `qbuf` holds the rows of this sub-tile on entry and, once they are parked in LDS, takes the rows
  // of the sub-tile after the next (token ids tok_next): the gathers of two sub-tiles are in flight at a time
  auto step = [&](vec8 (&qbuf)[NLD], int token, int sub, int tok_next) {
    const int r = sub + col;
    const bool valid = r < row_hi;
    if (STAGED) {
#pragma unroll
      for (int j = 0; j < NLD; ++j) store16(&Ost[(srow + RPI * j) * OS + schunk * 8], qbuf[j]);
      __builtin_amdgcn_wave_barrier();
      if (sub + 2 * SEL_WG_ROWS < row_hi) fetch_q(qbuf, tok_next, sub + 2 * SEL_WG_ROWS);
    }
    f32x16 acc[NA];
#pragma unroll
    for (int a = 0; a < NA; ++a) {
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        vec8 kf = load16<vec8>(&Ks[(a * 32 + col) * KS + (STAGED ? hh * (D / 2) + ks * 8 : ks * 16 + hh * 8)]);
        vec8 qf = STAGED ? load16<vec8>(&Ost[col * OS + hh * (D / 2) + ks * 8]) : qdir[STAGED ? 0 : ks];
        acc[a] = Elem<T>::mfma32(kf, qf, acc[a]);
      }
    }
    __builtin_amdgcn_wave_barrier();  // Q fragments consumed: the tile is reused for the output rows
    if (!STAGED && sub + SEL_WG_ROWS < row_hi) fetch_dir(tok_next, sub + SEL_WG_ROWS);
    // causal mask: key index inside the block must be <= limit
    const int limit = (token - seq_start) - b_local * BK;
    float mx = -INFINITY;
    // only the rows of the block's own queries see it partly: a wave without such a row skips the mask
    if (!__all(limit >= BK - 1)) {
#pragma unroll
      for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = a * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
          if (key > limit) acc[a][i] = -INFINITY;
        }
    }
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, acc[a][i]);
    mx = fmaxf(mx, xor32(mx));
    const float mref = (mx == -INFINITY) ? 0.f : mx * p.scale_log2;
    float l = 0.f;
    vec8 pk[NJ];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pv = fast_exp2(acc[a][i] * p.scale_log2 - mref);
        l += pv;
        pk[a * 2 + (i >> 3)][i & 7] = (T)pv;
      }
    l += xor32(l);
    const float inv_l = l > 0.f ? 1.f / l : 0.f;
    const int64_t prow = prow0 + r;
    // O^T accumulators -> this wave's LDS tile [row][d] -> 16-byte stores in which 16 lanes
    // cover one full 2*D-byte row (8 cache lines per store instruction instead of 64)
    // the products of the next 32 dims are issued before the current ones are converted and stored: the matrix
    // unit works on them while the vector unit, the LDS and the stores deal with the finished accumulator
    auto pv = [&](int dt) {
      f32x16 acc_;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc_[i] = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        vec8 vf = lds_read_tr8<T>(vtr + 16 * j * VS + dt * 32, 8 * VS);
        acc_ = Elem<T>::mfma32(vf, pk[j], acc_);
      }
      return acc_;
    };
    f32x16 onext = pv(0);
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const f32x16 oacc = onext;
      if (dt + 1 < NDT) onext = pv(dt + 1);
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        typename Elem<T>::vec4 x;
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = (T)(oacc[4 * qd + e] * inv_l);
        if (SelLds<D, BK>::STAGE_OUT) store8(&Ost[col * OS + dt * 32 + 8 * qd + 4 * hh], x);
        else if (SelLds<D, BK>::SLICE_OUT) store8(&Osl[col * SLS + 8 * qd + 4 * hh], x);
        else if (valid) store8(opart + prow * D + dt * 32 + 8 * qd + 4 * hh, x);  // LDS too small: direct
      }
      if (SelLds<D, BK>::SLICE_OUT) {  // the 32 dims of this accumulator: 4 lanes per row, 16 rows per store
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int row = (lane >> 2) + 16 * j;
          vec8 y = load16<vec8>(&Osl[row * SLS + (lane & 3) * 8]);
          // 64-byte pieces: left to the L2 to merge into whole lines (as non-temporal stores they cost 4 % more)
          if (sub + row < row_hi) store16(opart + (prow0 + sub + row) * D + dt * 32 + (lane & 3) * 8, y);
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
    __builtin_amdgcn_wave_barrier();
    if (SelLds<D, BK>::STAGE_OUT) {
      constexpr int CPR = D / 8;          // 16-byte chunks per row
      constexpr int RPI = 64 / CPR;       // rows per store instruction
      const int srow = lane / CPR, schunk = lane % CPR;
#pragma unroll
      for (int j = 0; j < 32 / RPI; ++j) {
        const int row = srow + RPI * j;
        vec8 x = load16<vec8>(&Ost[row * OS + schunk * 8]);
        if (sub + row < row_hi) store16_stream(opart + (prow0 + sub + row) * D + schunk * 8, x);
      }
    }
    __builtin_amdgcn_wave_barrier();
    if (valid && hh == 0) __builtin_nontemporal_store(l > 0.f ? mref + log2f(l) : -INFINITY, &p.lse_part[prow]);
  };

  int sub = row_lo + wv * 32;
  if (sub >= row_hi) return;
  int ta = row_token(sub);
  if (STAGED) {
    auto tok_at = [&](int s_) { return s_ < row_hi ? row_token(s_) : 0; };
    int tb = tok_at(sub + SEL_WG_ROWS), tc = tok_at(sub + 2 * SEL_WG_ROWS), td = tok_at(sub + 3 * SEL_WG_ROWS);
    fetch_q(qst, ta, sub);
    if (sub + SEL_WG_ROWS < row_hi) fetch_q(qst_b, tb, sub + SEL_WG_ROWS);
    for (;;) {  // two sub-tiles per round, one from each buffer
      const int te = tok_at(sub + 4 * SEL_WG_ROWS), tf = tok_at(sub + 5 * SEL_WG_ROWS);
      step(qst, ta, sub, tc);
      if (sub + SEL_WG_ROWS >= row_hi) break;
      step(qst_b, tb, sub + SEL_WG_ROWS, td);
      sub += 2 * SEL_WG_ROWS;
      if (sub >= row_hi) break;
      ta = tc; tb = td; tc = te; td = tf;
    }
    return;
  }
  fetch_dir(ta, sub);
  int tb = sub + SEL_WG_ROWS < row_hi ? row_token(sub + SEL_WG_ROWS) : 0;
  for (; sub < row_hi; sub += SEL_WG_ROWS) {
    const int tc = sub + 2 * SEL_WG_ROWS < row_hi ? row_token(sub + 2 * SEL_WG_ROWS) : 0;
    step(qst, ta, sub, tb);
    ta = tb;
    tb = tc;
  }
}

// Query-major merge.  D/8 lanes own one (query, head) row, 16 bytes each.
template <typename T, int D>
__global__ void __launch_bounds__(256)
selattn_fwd_reduce_kernel(const T* __restrict__ o_part, const float* __restrict__ lse_part,
                          const int32_t* __restrict__ slot_of, int64_t cap, int64_t n_tokens, int hq,
                          int g, int topk, T* __restrict__ o, int64_t o_sn, int64_t o_sh,
                          float* __restrict__ lse) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int LPR = D / 8;
  constexpr int RPB = 256 / LPR;
  const int64_t R = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
  const int sub = threadIdx.x % LPR;
  if (R >= n_tokens * hq) return;
  const int64_t tok = R / hq;
  const int hq_i = (int)(R - tok * hq);
  const int kh = hq_i / g, head = hq_i - kh * g;
  const int32_t* so = slot_of + ((int64_t)kh * n_tokens + tok) * topk;
  const int64_t pbase = (int64_t)kh * cap;

  // The LPR lanes of a row split the slots: lane `sub` owns slots sub, sub + LPR, ...  Position and partial LSE of
  // a slot are loaded once by their owner and handed to the other lanes by shuffles.
  constexpr int MAXC = 8;  // chunks of LPR slots kept in registers (topk <= 8 * LPR; more are re-read)
  const int nchunk = (topk + LPR - 1) / LPR;
  int pidx_c[MAXC];
  float lse_c[MAXC];
  float mx = -INFINITY;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    pidx_c[c] = -1;
    lse_c[c] = -INFINITY;
    if (c < nchunk) {
      const int t = c * LPR + sub;
      if (t < topk) pidx_c[c] = so[t];
      if (pidx_c[c] >= 0) lse_c[c] = lse_part[(pbase + pidx_c[c]) * g + head];
      mx = fmaxf(mx, lse_c[c]);
    }
  }
  for (int t = MAXC * LPR + sub; t < topk; t += LPR) {  // beyond the register chunks
    const int pidx = so[t];
    if (pidx >= 0) mx = fmaxf(mx, lse_part[(pbase + pidx) * g + head]);
  }
#pragma unroll
  for (int o_ = LPR / 2; o_ >= 1; o_ >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o_, LPR));
  float sum = 0.f;
  if (mx > -INFINITY) {
#pragma unroll
    for (int c = 0; c < MAXC; ++c)
      if (c < nchunk) sum += fast_exp2(lse_c[c] - mx);  // -inf -> 0
    for (int t = MAXC * LPR + sub; t < topk; t += LPR) {
      const int pidx = so[t];
      if (pidx >= 0) sum += fast_exp2(lse_part[(pbase + pidx) * g + head] - mx);
    }
  }
#pragma unroll
  for (int o_ = LPR / 2; o_ >= 1; o_ >>= 1) sum += __shfl_xor(sum, o_, LPR);
  const float lse_tot = sum > 0.f ? mx + log2f(sum) : -INFINITY;

  // weighted sum of the partial rows
  float accv[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) accv[e] = 0.f;
  if (sum > 0.f) {
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nchunk) {  // uniform
        const float w_mine = fast_exp2(lse_c[c] - lse_tot);  // 0 for padding slots
#pragma unroll
        for (int j = 0; j < LPR; ++j) {
          const int pidx = __shfl(pidx_c[c], j, LPR);
          const float wgt = __shfl(w_mine, j, LPR);
          if (pidx >= 0) {
            const int64_t prow = (pbase + pidx) * g + head;
            vec8 x = load16_stream<vec8>(o_part + prow * D + sub * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e) accv[e] += wgt * (float)x[e];
          }
        }
      }
    }
    for (int t = MAXC * LPR; t < topk; ++t) {
      const int pidx = so[t];
      if (pidx < 0) continue;
      const int64_t prow = (pbase + pidx) * g + head;
      const float wgt = fast_exp2(lse_part[prow] - lse_tot);
      vec8 x = load16_stream<vec8>(o_part + prow * D + sub * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) accv[e] += wgt * (float)x[e];
    }
  }
  vec8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (T)accv[e];
  store16_stream(o + tok * o_sn + (int64_t)hq_i * o_sh + sub * 8, out);
  if (sub == 0) lse[(int64_t)hq_i * n_tokens + tok] = lse_tot;
}

struct FwdWs {
  size_t off_opart, off_lse, off_tiles, off_tile_block, total;
  int64_t max_tiles;
};

// bk <= 0: the block size is not known (workspace query): room for the smallest tiles any block size uses
static FwdWs fwd_ws_layout(int64_t n_tokens, int hq, int hkv, int d, int topk, int bk, int64_t max_blocks) {
  FwdWs w;
  const int g = hq / hkv;
  const size_t cap = (size_t)n_tokens * topk;
  w.off_opart = 0;
  w.off_lse = align_up(cap * hkv * g * d * 2, 256);
  w.off_tiles = w.off_lse + align_up(cap * hkv * g * 4, 256);
  w.off_tile_block = w.off_tiles + align_up((size_t)hkv * (max_blocks + 1) * 4, 256);
  w.max_tiles = fsa_max_tiles(n_tokens, topk, g, bk > 0 ? sel_tile_rows(g, d, bk) : 1024, max_blocks);
  w.total = w.off_tile_block + align_up((size_t)hkv * fsa_max_tiles(n_tokens, topk, g, 1024, max_blocks) * 4, 256);
  return w;
}

template <typename T, int D, int BK>
static int launch_main(const SelFwdParams& p, int hkv, int64_t max_tiles, hipStream_t stream) {
  constexpr int lds = SelLds<D, BK>::BYTES;
  static bool attr_done = false;
  if (!attr_done && lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)selattn_fwd_main_kernel<T, D, BK>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) {
      set_error("hipFuncSetAttribute(%d B LDS): %s", lds, hipGetErrorString(e));
      return (int)e;
    }
    attr_done = true;
  }
  dim3 grid((unsigned)max_tiles, hkv);
  ProfScope ps_("selattn_fwd_main", stream);
  selattn_fwd_main_kernel<T, D, BK><<<grid, SelLds<D, BK>::THREADS, lds, stream>>>(p);
  return 0;
}

template <typename T>
static int dispatch_main(int d, int bk, const SelFwdParams& p, int hkv, int64_t max_tiles,
                         hipStream_t stream) {
#define FSA_CASE(DD, BB) \
  if (d == DD && bk == BB) return launch_main<T, DD, BB>(p, hkv, max_tiles, stream);
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
  set_error("selected attention: head_dim=%d with block_size=%d is not supported "
            "(head_dim in {64,128,256}, block_size in {32,64,128})", d, bk);
  return FSA_ERR_UNSUPPORTED;
}

template <typename T>
static int launch_reduce(int d, const void* o_part, const float* lse_part, const int32_t* slot_of,
                         int64_t cap, int64_t n, int hq, int g, int topk, void* o, int64_t o_sn,
                         int64_t o_sh, float* lse, hipStream_t stream) {
  const int64_t rows = n * hq;
#define FSA_CASE(DD)                                                                          \
  if (d == DD) {                                                                              \
    constexpr int RPB = 256 / (DD / 8);                                                       \
    ProfScope ps_("selattn_fwd_reduce", stream);                                              \
    selattn_fwd_reduce_kernel<T, DD><<<(unsigned)((rows + RPB - 1) / RPB), 256, 0, stream>>>( \
        (const T*)o_part, lse_part, slot_of, cap, n, hq, g, topk, (T*)o, o_sn, o_sh, lse);    \
    return 0;                                                                                 \
  }
  FSA_CASE(64)
  FSA_CASE(128)
  FSA_CASE(256)
#undef FSA_CASE
  set_error("selected attention reduce: head_dim=%d not supported", d);
  return FSA_ERR_UNSUPPORTED;
}

}  // namespace fsa

using namespace fsa;

extern "C" size_t fsa_selattn_fwd_workspace_bytes(int64_t total_tokens, int32_t num_q_heads,
                                                  int32_t num_kv_heads, int32_t head_dim, int32_t topk,
                                                  int64_t max_blocks) {
  return fwd_ws_layout(total_tokens, num_q_heads, num_kv_heads, head_dim, topk, 0, max_blocks).total;
}

extern "C" int fsa_selattn_fwd(const void* q, const void* k, const void* v, int32_t dtype,
                               int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n,
                               int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                               const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens,
                               int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                               int32_t topk, int32_t block_size, int64_t max_blocks,
                               float softmax_scale, const int32_t* cu_blocks, const int32_t* counts,
                               const int32_t* starts, const int32_t* sel_tokens,
                               const int32_t* slot_of, void* o, int64_t o_stride_n,
                               int64_t o_stride_h, float* lse, void* workspace,
                               size_t workspace_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(q && k && v && o && lse && cu_seqlens && cu_blocks && counts && starts && sel_tokens &&
                    slot_of, "fsa_selattn_fwd: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_selattn_fwd: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(num_kv_heads >= 1 && num_q_heads % num_kv_heads == 0,
                "fsa_selattn_fwd: num_q_heads must be a multiple of num_kv_heads");
  FSA_CHECK_ARG(batch >= 1 && total_tokens >= 1 && topk >= 1, "fsa_selattn_fwd: empty problem");
  FSA_CHECK_ARG(total_tokens * topk < ((int64_t)1 << 31), "fsa_selattn_fwd: total_tokens*topk >= 2^31");
  FSA_CHECK_ARG((q_stride_n | q_stride_h | k_stride_n | k_stride_h | v_stride_n | v_stride_h |
                 o_stride_n | o_stride_h) % 8 == 0,
                "fsa_selattn_fwd: strides must be multiples of 8 elements (16-byte rows)");
  const int g = num_q_heads / num_kv_heads;
  // the kernels form q row addresses with 32-bit strides
  FSA_CHECK_ARG(q_stride_n >= 0 && q_stride_n < ((int64_t)1 << 31) && q_stride_h >= 0 &&
                    g * q_stride_h + head_dim < ((int64_t)1 << 31),
                "fsa_selattn_fwd: q strides too large or negative");
  FwdWs ws = fwd_ws_layout(total_tokens, num_q_heads, num_kv_heads, head_dim, topk, block_size, max_blocks);
  if (!workspace || workspace_bytes < ws.total) {
    set_error("fsa_selattn_fwd: workspace too small (%zu < %zu)", workspace_bytes, ws.total);
    return FSA_ERR_WORKSPACE;
  }
  char* wsp = (char*)workspace;
  int32_t* tile_prefix = (int32_t*)(wsp + ws.off_tiles);
  int32_t* tile_block = (int32_t*)(wsp + ws.off_tile_block);
  const int64_t max_tiles = ws.max_tiles;
  int rc = build_tiles(counts, num_kv_heads, max_blocks, g, sel_tile_rows(g, head_dim, block_size), tile_prefix,
                       tile_block, max_tiles, stream);
  if (rc) return rc;

  SelFwdParams p;
  p.q = q; p.k = k; p.v = v;
  p.q_sn = q_stride_n; p.q_sh = q_stride_h;
  p.k_sn = k_stride_n; p.k_sh = k_stride_h;
  p.v_sn = v_stride_n; p.v_sh = v_stride_h;
  p.cu_seqlens = cu_seqlens; p.cu_blocks = cu_blocks; p.counts = counts; p.starts = starts;
  p.sel_tokens = sel_tokens; p.tile_prefix = tile_prefix; p.tile_block = tile_block; p.max_tiles = max_tiles;
  p.batch = batch; p.max_blocks = max_blocks; p.cap = total_tokens * topk; p.g = g;
  p.g_shift = group_shift(g);

  p.scale_log2 = softmax_scale * LOG2E;
  p.o_part = wsp + ws.off_opart;
  p.lse_part = (float*)(wsp + ws.off_lse);

  rc = dtype == FSA_BF16
           ? dispatch_main<__bf16>(head_dim, block_size, p, num_kv_heads, max_tiles, stream)
           : dispatch_main<_Float16>(head_dim, block_size, p, num_kv_heads, max_tiles, stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_selattn_fwd main");
  rc = dtype == FSA_BF16
           ? launch_reduce<__bf16>(head_dim, p.o_part, p.lse_part, slot_of, p.cap, total_tokens,
                                   num_q_heads, g, topk, o, o_stride_n, o_stride_h, lse, stream)
           : launch_reduce<_Float16>(head_dim, p.o_part, p.lse_part, slot_of, p.cap, total_tokens,
                                     num_q_heads, g, topk, o, o_stride_n, o_stride_h, lse, stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_selattn_fwd reduce");
  return 0;
}
