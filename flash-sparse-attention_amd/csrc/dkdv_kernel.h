// dK/dV kernel shared by selected attention (gathered query rows of a kv block)
// and compressed attention (the dense range of queries that can see a tile of
// compressed keys).  Block-major, contraction over the rows: each wave owns 16
// keys and keeps their K / V fragments in registers; Q / dO tiles of 64 rows go
// through LDS once and feed S = Q K^T, dP = dO V^T (16x16x32 MFMA) and, through
// transposing LDS reads, dV^T += dO^T P and dK^T += Q^T dS.  The g heads of a
// group are rows of the same tile, so the results are already summed over the
// group, in fp32.  A block whose rows span several work-groups writes fp32
// partials that the reduce kernel adds in a fixed order.
#pragma once
#include "fsa_common.h"

#include <type_traits>

namespace fsa {

struct SelBwdParams {
  const void* q;
  const void* k;
  const void* v;
  const void* d_o;
  const float* lse;    // [Hq, N]
  const float* delta;  // [Hq, N]
  // selected mode: (lse, delta) pairs [N, Hq] instead of the two arrays above - the rows of a block are scattered
  // queries, and the statistics of a query's g heads then share one 8 g byte piece of a line instead of 2 g lines
  const float2* stat2;
  int hq;              // q heads in all (selected mode)
  int64_t q_sn, q_sh, k_sn, k_sh, v_sn, v_sh, do_sn, do_sh;
  const int32_t* cu_seqlens;
  const int32_t* cu_blocks;
  const int32_t* counts;
  const int32_t* starts;
  const int32_t* sel_tokens;
  const int32_t* tile_prefix;
  const int32_t* tile_block;  // [Hkv, max_tiles]: block of every tile, or null (binary search through tile_prefix)
  int batch;
  int64_t max_blocks;
  int64_t cap;
  int64_t n_tokens;
  int g;
  int g_shift;  // log2 g, or -1 if g is not a power of two
  float scale;
  float scale_log2;
  void* dq_part;     // [Hkv, cap, g, D]
  float* dkdv_part;  // [Hkv, max_tiles, 2, BK, D]
  int64_t max_tiles;
  int kv_tile_rows;  // rows per work-group of the dK/dV kernel
  void* dk;          // rows of k's shape, strides dk_sn / dk_sh
  void* dv;
  int64_t dk_sn, dk_sh;
  // compressed-attention mode only
  const int32_t* cu_seqlens_k;
  int kernel_size, kernel_stride;
  int window;  // sliding-window mode only
};

// Host: the kernels form q / dO row addresses with 32-bit strides - token stride and the whole span of a kv head's
// q heads must be non-negative and below 2^31 elements.
inline bool kv_qdo_strides_ok(int64_t q_sn, int64_t q_sh, int64_t do_sn, int64_t do_sh, int g, int head_dim) {
  const int64_t lim = (int64_t)1 << 31;
  return q_sn >= 0 && q_sn < lim && do_sn >= 0 && do_sn < lim && q_sh >= 0 && do_sh >= 0 &&
         g * q_sh + head_dim < lim && g * do_sh + head_dim < lim;
}

constexpr int KV_REDUCE_SPLIT = 32;  // work-groups that share the blocks of one span in the dK/dV reduce kernel
constexpr int KV_REDUCE_SPAN = 64;   // blocks examined by one work-group of that kernel
constexpr int KV_MODE_SELECTED = 0;
constexpr int KV_MODE_COMPRESSED = 1;
constexpr int KV_MODE_WINDOW = 2;  // sliding window: key p visible to query i iff i - window <= p <= i

// What a "block" of the work list is in each mode.
template <int MODE, int BK> struct KvBlock {
  int seq_start, q_first, key_row0, n_keys_valid, key_base;
  __device__ __forceinline__ void init(const SelBwdParams& p, int gb) {
    const int s = upper_seg(p.cu_blocks, p.batch, gb);
    const int b_local = gb - p.cu_blocks[s];
    seq_start = p.cu_seqlens[s];
    if (MODE == KV_MODE_SELECTED) {
      key_row0 = seq_start + b_local * BK;                 // K/V rows are tokens
      n_keys_valid = p.cu_seqlens[s + 1] - key_row0;       // may exceed BK
      q_first = 0;
      key_base = b_local * BK;                             // position of key 0 of the block
    } else if (MODE == KV_MODE_WINDOW) {
      key_row0 = seq_start + b_local * BK;
      n_keys_valid = p.cu_seqlens[s + 1] - key_row0;
      q_first = b_local * BK;                              // a key is first seen by the query at its own position
      key_base = b_local * BK;
    } else {
      const int k0 = p.cu_seqlens_k[s];
      key_row0 = k0 + b_local * BK;                        // K/V rows are compressed tokens
      n_keys_valid = p.cu_seqlens_k[s + 1] - key_row0;
      q_first = b_local * BK * p.kernel_stride + p.kernel_size - 1;  // first query that sees key 0
      key_base = b_local * BK;
    }
  }
  // number of keys of the block visible to the query at sequence-local position qpos, minus one
  __device__ __forceinline__ int limit(const SelBwdParams& p, int qpos) const {
    if (MODE == KV_MODE_SELECTED || MODE == KV_MODE_WINDOW) return qpos - key_base;
    return (qpos - p.kernel_size + 1) / p.kernel_stride - key_base;  // qpos >= q_first >= ks-1
  }
  // first key of the block (index inside the block) visible to that query
  __device__ __forceinline__ int limit_lo(const SelBwdParams& p, int qpos) const {
    if (MODE == KV_MODE_WINDOW) return qpos - p.window - key_base;
    return -(1 << 30);
  }
};

// ----------------------------------------------------------------- dkdv ----
// Upper bound of the rows one work-group takes from a block (a block with more rows is dealt in equal shares to
// several work-groups, which then write fp32 dK / dV partials): measured optimum 3072 / 5120 / 8192 rows for GQA
// groups of 1 / 2 / 4 - smaller tiles balance better, larger ones write fewer partials.
constexpr int KV_TILE_ROWS_MAX = 8192;
static inline int kv_tile_rows(int g, int d = 128, int bk = 64) {
  if (d >= 256 && bk >= 128) return KV_TILE_ROWS_MAX;  // 32-row passes of eight waves: fewer, longer tiles
  const int r = 1024 + 2048 * g;
  return r < KV_TILE_ROWS_MAX ? r : KV_TILE_ROWS_MAX;
}

// Element offset of element `col` (a multiple of 4) of row `row` in an unpadded LDS tile with rows of W 16-bit
// elements.  The LDS serves a half-wave (32 lanes) per cycle from 64 four-byte banks, so the 8-byte reads of a
// half-wave must fall into distinct 16-byte slots of the 256-byte bank line.  The two read patterns of the MFMA
// operands are 16 rows x 16 bytes (natural: row = lane % 16) and 8 rows x 32 bytes (transposing: four lanes per
// row); with rows that are a multiple (or a fraction) of 256 bytes both would hit the same slots in every row.
// Hence: the 32-byte group index of a row is XOR-ed with the row number (8 consecutive rows -> 8 different
// groups), and the two 16-byte halves of every group are swapped in rows 8..15 of each 16 (16 rows x 16 bytes ->
// 16 different slots).  Measured on gfx950 (ds_read_b64 / ds_read_b64_tr_b16, 8 waves per CU): both patterns at
// the full rate of 1.04 ns per wave instruction, where rows padded to 272 bytes give 1.04 / 1.86 (the
// transposing reads two-way conflicted) and rows of 288 bytes 1.86 / 1.04.
template <int W> __device__ __forceinline__ int swz(int row, int col) {
  static_assert(W >= 32 && (W & (W - 1)) == 0, "row length");
  constexpr int L = W >= 128 ? 1 : 128 / W;          // rows per 256-byte bank line
  constexpr int XM = W / 16 - 1 < 7 ? W / 16 - 1 : 7;  // 32-byte groups per row - 1, at most 8 take part
  const int x = (row / L) & XM, hb = (row >> 3) & 1;
  return row * W + ((((col >> 4) ^ x) << 4) | ((((col >> 3) & 1) ^ hb) << 3) | (col & 7));
}

template <int D, int BK> struct KvCfg {
  static constexpr int NW = BK / 16;        // one wave per 16 keys
  // gathered rows per pass; 32 where 8 waves of head_dim 256 leave no registers for a 64-row pass
  static constexpr int KV_R = (D >= 256 && BK >= 128) ? 32 : 64;
  static constexpr int NT = NW * 64;
  static constexpr int QS = D;             // LDS rows of the Q / dO tiles are unpadded and swizzled (swz<D>)
  static constexpr int CPR = D / 8;         // 16-byte chunks per row
  static constexpr int CPT = KV_R * CPR / NT;  // chunks per thread and tensor
  static constexpr int ROW_STEP = NT / CPR;
  static constexpr int BYTES = 2 * KV_R * QS * 2 + KV_R * 16;
  // with the fused dQ: K of the block (natural layout) and the dS^T tile [BK][KV_R]
  static constexpr int KS = D;            // K copy: unpadded and swizzled like the Q / dO tiles
  static constexpr int DSS = KV_R + 8;    // the small dS^T and dQ staging tiles keep padded rows
  // fused dQ: row tiles (16 rows) are dealt to the waves; with more waves than row tiles, TG waves share a
  // row tile and split its d tiles.  Each wave stages its [16][DW] piece for row-coalesced stores.
  static constexpr int NRT = KV_R / 16;
  static constexpr int TG = NW > NRT ? NW / NRT : 1;
  static constexpr int RW = NW / TG;                 // waves that start on distinct row tiles
  static constexpr int DW = D / TG;                  // columns of dQ per wave
  static constexpr int DQS = DW + 8;
  static constexpr bool STAGE_DQ = BYTES + (BK * KS + BK * DSS + NW * 16 * DQS) * 2 <= 160 * 1024;
  static constexpr int BYTES_FUSED = BYTES + (BK * KS + BK * DSS + (STAGE_DQ ? NW * 16 * DQS : 0)) * 2;
  static constexpr int MIN_WAVES = (D <= 128 && NT <= 256) ? 2 : 1;  // work-groups per CU the registers allow
  // with 8 waves the register budget is 256 per lane: K fragments are then re-read from the LDS copy of the
  // block that the fused dQ keeps anyway, instead of living in 32 registers
  static constexpr bool K_FROM_LDS = D >= 256 && NT >= 512;
  static constexpr bool TIGHT_REGS = D >= 256 && NT >= 512;
  static_assert(KV_R * CPR % NT == 0, "tile must divide evenly over the threads");
};

// FUSE_DQ (selected mode): the work-group also produces the partial dQ rows of
// its (query, block) pairs - dQ^T = K^T dS^T with dS^T exchanged between the
// waves through LDS - so Q and dO are gathered once for dQ, dK and dV.
template <typename T, int D, int BK, int MODE, bool FUSE_DQ = false>
__global__ void __launch_bounds__((KvCfg<D, BK>::NT), (KvCfg<D, BK>::MIN_WAVES))
attn_bwd_dkdv_kernel(SelBwdParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef typename Elem<T>::vec4 vec4;
  typedef KvCfg<D, BK> C;
  constexpr int QS = C::QS, NS = D / 32, NDT = D / 16, NRT = C::NRT, NU = C::KV_R / 32;
  // aligned to the bank line and to the largest swizzled row: group addresses are formed by XOR on byte addresses
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  T* Qs = reinterpret_cast<T*>(smem);
  T* Os = Qs + C::KV_R * QS;
  float* lse_s = reinterpret_cast<float*>(Os + C::KV_R * QS);
  float* del_s = lse_s + C::KV_R;
  int* lim_s = reinterpret_cast<int*>(del_s + C::KV_R);
  int* llo_s = lim_s + C::KV_R;
  T* Kl = reinterpret_cast<T*>(llo_s + C::KV_R);   // FUSE_DQ only
  T* dSs = Kl + BK * C::KS;                     // FUSE_DQ only
  T* dQst = dSs + BK * C::DSS + (threadIdx.x >> 6) * (16 * C::DQS);  // FUSE_DQ only: this wave's [16][DW] tile

  const int h = blockIdx.y;
  const int64_t nbp1 = p.max_blocks + 1;
  const int32_t* tp = p.tile_prefix + h * nbp1;
  const int w = blockIdx.x;
  if (w >= tp[p.max_blocks]) return;
  const int gb = p.tile_block ? p.tile_block[h * p.max_tiles + w] : upper_seg(tp, (int)p.max_blocks, w);
  KvBlock<MODE, BK> blk;
  blk.init(p, gb);
  const int rows = p.counts[h * p.max_blocks + gb] * p.g;
  const int start = MODE == KV_MODE_SELECTED ? p.starts[h * nbp1 + gb] : 0;
  const int ntile_b = tp[gb + 1] - tp[gb];
  // the rows of the block are dealt to its work-groups in equal shares (whole passes): a full tile followed by a
  // short remainder, block after block, would put the long and the short tiles on alternating XCDs
  const int share = ((rows + ntile_b - 1) / ntile_b + C::KV_R - 1) / C::KV_R * C::KV_R;
  const int row_lo = (w - tp[gb]) * share;
  const int row_hi = min(rows, row_lo + share);

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int l16 = lane & 15, kg = lane >> 4;
  const int key = wv * 16 + l16;       // this lane's key inside the block (B operand column)
  const int ktok = blk.key_row0 + key;  // row of this lane's key in k / v
  const bool key_ok = key < blk.n_keys_valid;

  // K / V fragments of this wave's 16 keys stay in registers: B[k = d][n = key]
  constexpr bool KLDS = FUSE_DQ && C::K_FROM_LDS;
  // hand-issued 8-byte fragment reads (and the contraction-index mapping that goes with them) where the
  // registers allow it
  constexpr bool SPLIT = !KLDS && NS <= 4 && C::CPT <= 4;
  vec8 kf[KLDS ? 1 : NS], vf[NS];
  {
    // Contraction index of the S / dP products: k-step s_ covers dims [32 s_, 32 s_ + 32); the lane of key
    // group kg holds dims 4 kg .. 4 kg + 3 and 16 + 4 kg .. 16 + 4 kg + 3 of it.  Both halves are 8-byte
    // pieces, so the matching Q / dO fragments come from LDS with 8-byte reads in which the four key groups
    // read 32 contiguous bytes of a row (full LDS rate; a 16-byte read per lane runs at half of it).
    // (Configurations that keep the compiler-issued 16-byte reads - SPLIT false - use the plain mapping: dims
    // 8 kg .. 8 kg + 7 of the k-step.)
    const T* krow = reinterpret_cast<const T*>(p.k) + (int64_t)ktok * p.k_sn + (int64_t)h * p.k_sh + (SPLIT ? 4 : 8) * kg;
    const T* vrow = reinterpret_cast<const T*>(p.v) + (int64_t)ktok * p.v_sn + (int64_t)h * p.v_sh + (SPLIT ? 4 : 8) * kg;
#pragma unroll
    for (int s_ = 0; s_ < NS; ++s_) {
      if (!KLDS) kf[s_] = zero8<T>();
      vf[s_] = zero8<T>();
      if (key_ok) {
        if (!KLDS) kf[s_] = SPLIT ? load8x2<T>(krow + 32 * s_) : load16<vec8>(krow + 32 * s_);
        vf[s_] = SPLIT ? load8x2<T>(vrow + 32 * s_) : load16<vec8>(vrow + 32 * s_);
      }
    }
  }

  if (FUSE_DQ) {
    const T* kb = reinterpret_cast<const T*>(p.k) + (int64_t)h * p.k_sh;
    for (int c = tid; c < BK * (D / 8); c += C::NT) {
      const int row = c / (D / 8), cc = c % (D / 8);
      vec8 x = zero8<T>();
      if (row < blk.n_keys_valid) x = load16<vec8>(kb + (int64_t)(blk.key_row0 + row) * p.k_sn + cc * 8);
      store16(&Kl[swz<D>(row, cc * 8)], x);
    }
  }
  const int32_t* toks = MODE == KV_MODE_SELECTED ? p.sel_tokens + (int64_t)h * p.cap + start : nullptr;
  // row r of the block -> global query row
  auto row_token = [&](int r) {
    if (MODE == KV_MODE_SELECTED) return (int)toks[div_group(r, p.g, p.g_shift)];
    return blk.seq_start + blk.q_first + div_group(r, p.g, p.g_shift);
  };
  const T* qbase = reinterpret_cast<const T*>(p.q) + (int64_t)h * p.g * p.q_sh;
  const T* dobase = reinterpret_cast<const T*>(p.d_o) + (int64_t)h * p.g * p.do_sh;
  const int ld_row = tid / C::CPR, ld_col = tid % C::CPR;
  const uint32_t q_sn32 = (uint32_t)p.q_sn, q_sh32 = (uint32_t)p.q_sh, do_sn32 = (uint32_t)p.do_sn, do_sh32 = (uint32_t)p.do_sh;

  vec8 qst[C::CPT], dost[C::CPT];
  float lse_st = 0.f, del_st = 0.f;
  int lim_st = 0, llo_st = 0;
  int tok_pf[C::CPT], tok_stat = 0;  // token ids of the pass after the one being fetched
  auto fetch_tokens = [&](int base) {
#pragma unroll
    for (int j = 0; j < C::CPT; ++j) {
      // rows past the end of the share repeat its last row (see fetch)
      const int r = max(min(base + ld_row + C::ROW_STEP * j, row_hi - 1), 0);
      tok_pf[j] = row_token(r);
    }
    if (tid < C::KV_R) tok_stat = base + tid < row_hi ? row_token(base + tid) : 0;
  };
  // global -> registers for the pass starting at row `base` (its token ids are in tok_pf)
  auto fetch = [&](int base) {
#pragma unroll
    for (int j = 0; j < C::CPT; ++j) {
      // row address = token * row stride + head * head stride + column: strides and the head term fit 32 bits
      // (checked by the host), so each address is one 32 x 32 -> 64 bit multiply-add.  Rows past the end of the
      // share repeat its last row - values of this block's own rows, which lse = +inf turns into P = dS = 0.
      const int r = max(min(base + ld_row + C::ROW_STEP * j, row_hi - 1), 0);
      const uint32_t head = p.g_shift >= 0 ? (uint32_t)(r & (p.g - 1)) : (uint32_t)(r - div_group(r, p.g, p.g_shift) * p.g);
      const uint32_t token = (uint32_t)tok_pf[j];
      qst[j] = load16<vec8>(qbase + ((uint64_t)token * q_sn32 + (head * q_sh32 + ld_col * 8)));
      dost[j] = load16<vec8>(dobase + ((uint64_t)token * do_sn32 + (head * do_sh32 + ld_col * 8)));
    }
    if (tid < C::KV_R) {
      const int r = base + tid;
      lse_st = INFINITY;  // rows past the end: P = exp2(s - inf) = 0
      del_st = 0.f;
      lim_st = -1;
      llo_st = 0;
      if (r < row_hi) {
        const int trank = div_group(r, p.g, p.g_shift), head = r - trank * p.g;
        const int token = tok_stat;
        // token ids are 32-bit, so n_tokens < 2^31: one 32 x 32 -> 64 bit multiply-add
        if (MODE == KV_MODE_SELECTED) {
          const float2 s2 = p.stat2[(uint64_t)(uint32_t)token * (uint32_t)p.hq + (uint32_t)(h * p.g + head)];
          lse_st = s2.x;
          del_st = s2.y;
        } else {
          const uint64_t stat = (uint64_t)(uint32_t)(h * p.g + head) * (uint32_t)p.n_tokens + (uint32_t)token;
          lse_st = p.lse[stat];
          del_st = p.delta[stat];
        }
        lim_st = blk.limit(p, token - blk.seq_start);
        llo_st = blk.limit_lo(p, token - blk.seq_start);
      }
    }
  };
  const int st_off = swz<D>(ld_row, ld_col * 8);
  auto stash = [&]() {
#pragma unroll
    for (int j = 0; j < C::CPT; ++j) {
      // the swizzle of a row repeats every 16 rows
      const int off = C::ROW_STEP % 16 == 0 ? st_off + C::ROW_STEP * j * QS : swz<D>(ld_row + C::ROW_STEP * j, ld_col * 8);
      store16(&Qs[off], qst[j]);
      store16(&Os[off], dost[j]);
    }
    if (tid < C::KV_R) {
      lse_s[tid] = lse_st;
      del_s[tid] = del_st;
      lim_s[tid] = lim_st;
      llo_s[tid] = llo_st;
    }
  };

  f32x4 dkacc[NDT], dvacc[NDT];
#pragma unroll
  for (int t = 0; t < NDT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dkacc[t][i] = 0.f;
      dvacc[t][i] = 0.f;
    }

  // lane addresses: A operand rows (natural) and transposing reads
  // The row part of a swizzled offset repeats every 16 rows and the 32-byte group g of a row sits at the
  // offset of group 0 XOR 16 g elements, so a lane keeps one offset per access pattern:
  // byte addresses inside the Q tile, 32-byte group 0: the row part of a swizzled offset repeats every 16 rows,
  // and group g of a row sits at the address of group 0 XOR 32 g (the tiles start on multiples of the row size)
  const uint32_t a_addr00 = lds_addr(Qs + swz<D>(l16, (SPLIT ? 4 : 8) * kg));            // + rt*16 rows
  const uint32_t tr_addr00 = lds_addr(Qs + swz<D>(4 * kg + (l16 >> 2), 4 * (l16 & 3)));  // + 32*u rows (+ 16 rows)
  constexpr int ROW_BYTES = QS * 2, O_BYTES = C::KV_R * ROW_BYTES;                        // Os - Qs
  constexpr int K_BYTES = 2 * O_BYTES + C::KV_R * 16;                                     // Kl - Qs


  fetch_tokens(row_lo);
  fetch(row_lo);
  fetch_tokens(row_lo + C::KV_R);
  stash();
  __syncthreads();
  for (int base = row_lo; base < row_hi; base += C::KV_R) {
    const bool more = base + C::KV_R < row_hi;
    // The per-group offsets (offset of group 0 XOR a constant) are formed where they are used: computed once
    // before the loop they would occupy some twenty registers for the whole kernel.
    uint32_t a_addr0 = a_addr00, tr_addr0 = tr_addr00;
    asm volatile("" : "+v"(a_addr0), "+v"(tr_addr0));
    if (more) {
      fetch(base + C::KV_R);
      fetch_tokens(base + 2 * C::KV_R);
    }

    vec4 pk[NRT], dsk[NRT];
    // Q / dO fragments of row tile rt: [Q lo s_ | Q hi s_ | dO lo s_ | dO hi s_], issued one row tile ahead
    constexpr bool RAW = SPLIT;
    constexpr int NF = RAW ? 4 * NS : 1;
    u32x2 fr[2][NF];
    // statistics of the lane's four rows of the tile: [lse 0-1 | lse 2-3 | delta 0-1 | delta 2-3 | limit 0-1 |
    // limit 2-3 (| lower limit 0-1 | 2-3 in window mode)]
    constexpr int NST = RAW ? (MODE == KV_MODE_WINDOW ? 8 : 6) : 1;
    u32x2 st[2][NST];
    const uint32_t s_addr = lds_addr(lse_s + 4 * kg);
    constexpr int STAT_BYTES = C::KV_R * 4;    // del_s - lse_s = lim_s - del_s = llo_s - lim_s
    // compiler-issued path: k-steps outside, row tiles inside, so that a K fragment that comes from LDS is read
    // once per pass
    f32x4 sacc_all[RAW ? 1 : NRT], dpacc_all[RAW ? 1 : NRT];
    if constexpr (!RAW) {
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt) {
        sacc_all[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
        dpacc_all[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int s_ = 0; s_ < NS; ++s_) {
        const vec8 kfrag = KLDS ? load16<vec8>(&Kl[swz<D>(key, 32 * s_ + 8 * kg)]) : kf[KLDS ? 0 : s_];
#pragma unroll
        for (int rt = 0; rt < NRT; ++rt) {
          vec8 qa = load16<vec8>(lds_ptr<T>((a_addr0 ^ (64u * s_)) + rt * 16 * ROW_BYTES));
          sacc_all[rt] = Elem<T>::mfma16(qa, kfrag, sacc_all[rt]);
          vec8 da = load16<vec8>(lds_ptr<T>((a_addr0 ^ (64u * s_)) + (O_BYTES + rt * 16 * ROW_BYTES)));
          dpacc_all[rt] = Elem<T>::mfma16(da, vf[s_], dpacc_all[rt]);
        }
        if (C::TIGHT_REGS && (s_ & 1) == 1) asm volatile("" ::: "memory");
      }
    }
    auto issue = [&](auto rt_c, u32x2 (&dst)[NF]) {
      constexpr int rt = decltype(rt_c)::value;
      if constexpr (RAW) {
        constexpr int RB = rt * 16 * QS * 2;
        u32x2 (&sd)[NST] = st[rt & 1];
#pragma unroll
        for (int a_ = 0; a_ < NST / 2; ++a_) {  // unrolled: the offsets below are constants
          if (a_ == 0) { sd[0] = lds_read8_raw<rt * 64>(s_addr); sd[1] = lds_read8_raw<rt * 64 + 8>(s_addr); }
          if (a_ == 1) { sd[2] = lds_read8_raw<STAT_BYTES + rt * 64>(s_addr); sd[3] = lds_read8_raw<STAT_BYTES + rt * 64 + 8>(s_addr); }
          if (a_ == 2) { sd[4] = lds_read8_raw<2 * STAT_BYTES + rt * 64>(s_addr); sd[5] = lds_read8_raw<2 * STAT_BYTES + rt * 64 + 8>(s_addr); }
          if (a_ == 3) { sd[NST - 2] = lds_read8_raw<3 * STAT_BYTES + rt * 64>(s_addr); sd[NST - 1] = lds_read8_raw<3 * STAT_BYTES + rt * 64 + 8>(s_addr); }
        }
        uint32_t a_addr = a_addr0;
        asm volatile("" : "+v"(a_addr));  // the group addresses are formed per row tile, next to their reads
#pragma unroll
        for (int s_ = 0; s_ < NS; ++s_) {  // group 2 s_ holds the first, group 2 s_ + 1 the second half of k-step s_
          const uint32_t lo = a_addr ^ (64u * s_), hi = a_addr ^ (64u * s_ + 32u);
          dst[s_] = lds_read8_raw<RB>(lo);
          dst[NS + s_] = lds_read8_raw<RB>(hi);
          dst[2 * NS + s_] = lds_read8_raw<O_BYTES + RB>(lo);
          dst[3 * NS + s_] = lds_read8_raw<O_BYTES + RB>(hi);
        }
      }
    };
    auto s_phase = [&](auto rt_c) {
      constexpr int rt = decltype(rt_c)::value;
      f32x4 sacc = {0.f, 0.f, 0.f, 0.f}, dpacc = {0.f, 0.f, 0.f, 0.f};
      if constexpr (RAW) {
        u32x2 (&cur)[NF] = fr[rt & 1];
        lds_wait<NF>(cur);
        lds_wait<NST>(st[rt & 1]);
        if constexpr (rt + 1 < NRT) issue(std::integral_constant<int, rt + 1>{}, fr[(rt + 1) & 1]);
#pragma unroll
        for (int s_ = 0; s_ < NS; ++s_) {
          sacc = Elem<T>::mfma16(frag8<T>(cur[s_], cur[NS + s_]), kf[KLDS ? 0 : s_], sacc);
          dpacc = Elem<T>::mfma16(frag8<T>(cur[2 * NS + s_], cur[3 * NS + s_]), vf[s_], dpacc);
        }
      } else {
        sacc = sacc_all[rt];
        dpacc = dpacc_all[rt];
      }
      float lse_r[4], del_r[4];
      int lim_r[4], llo_r[4] = {0, 0, 0, 0};
      if constexpr (RAW) {
        u32x2 (&sd)[NST] = st[rt & 1];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          lse_r[i] = __uint_as_float(sd[i >> 1][i & 1]);
          del_r[i] = __uint_as_float(sd[2 + (i >> 1)][i & 1]);
          lim_r[i] = (int)sd[4 + (i >> 1)][i & 1];
          if (MODE == KV_MODE_WINDOW) llo_r[i] = (int)sd[NST - 2 + (i >> 1)][i & 1];
        }
      } else {
        const float4 lse4 = *reinterpret_cast<const float4*>(&lse_s[rt * 16 + 4 * kg]);
        const float4 del4 = *reinterpret_cast<const float4*>(&del_s[rt * 16 + 4 * kg]);
        const int4 lim4 = *reinterpret_cast<const int4*>(&lim_s[rt * 16 + 4 * kg]);
        lse_r[0] = lse4.x; lse_r[1] = lse4.y; lse_r[2] = lse4.z; lse_r[3] = lse4.w;
        del_r[0] = del4.x; del_r[1] = del4.y; del_r[2] = del4.z; del_r[3] = del4.w;
        lim_r[0] = lim4.x; lim_r[1] = lim4.y; lim_r[2] = lim4.z; lim_r[3] = lim4.w;
        if (MODE == KV_MODE_WINDOW) {
          const int4 llo4 = *reinterpret_cast<const int4*>(&llo_s[rt * 16 + 4 * kg]);
          llo_r[0] = llo4.x; llo_r[1] = llo4.y; llo_r[2] = llo4.z; llo_r[3] = llo4.w;
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool vis = key <= lim_r[i] && (MODE != KV_MODE_WINDOW || key >= llo_r[i]);
        const float pv = vis ? fast_exp2(sacc[i] * p.scale_log2 - lse_r[i]) : 0.f;
        const float ds = pv * (dpacc[i] - del_r[i]) * p.scale;
        pk[rt][i] = (T)pv;
        dsk[rt][i] = (T)ds;
      }
    };
    issue(std::integral_constant<int, 0>{}, fr[0]);
    s_phase(std::integral_constant<int, 0>{});
    s_phase(std::integral_constant<int, 1>{});
    if constexpr (NRT > 2) {
      s_phase(std::integral_constant<int, 2>{});
      s_phase(std::integral_constant<int, 3>{});
    }
    static_assert(NRT == 2 || NRT == 4, "row tiles per pass");
    if (FUSE_DQ) {
      // dS^T[key][row] for the whole tile: every lane owns 4 consecutive rows of its key
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt) store8(&dSs[key * C::DSS + rt * 16 + 4 * kg], dsk[rt]);
      // (the other waves read it in the dQ products only: the barrier stands behind the dK / dV products, which
      // use the wave's own P and dS, so that a wave that is ahead does not wait here)
    }
    // The two waves of a SIMD are in different phases most of the time.  From here to the end of the pass the wave
    // issues its matrix products back to back (dK / dV, then dQ): raised priority keeps the other wave's vector work
    // from delaying them, and that wave fills the gaps (measured: fused backward -2 to -4 %; raising it for the
    // S / dP phase as well, or only for dK / dV, gains nothing).
    if (FUSE_DQ) __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      vec8 pb = __builtin_shufflevector(pk[2 * u], pk[2 * u + 1], 0, 1, 2, 3, 4, 5, 6, 7);
      vec8 dsb = __builtin_shufflevector(dsk[2 * u], dsk[2 * u + 1], 0, 1, 2, 3, 4, 5, 6, 7);
      // The operands of d tile t + 1 are requested before the products of d tile t are issued, one tile ahead and no
      // more: left to itself the compiler fetches the whole second half of the rows ahead (64 registers) and then
      // waits for each operand of the first half right after requesting it.
      auto rd = [&](int t, int which) {
        const T* trp = lds_ptr<T>(tr_addr0 ^ (32u * t));
        return lds_read_tr8<T>(trp + ((which ? O_BYTES / 2 : 0) + 32 * u * QS), 16 * QS);
      };
      if constexpr (D <= 128) {
        vec8 doa = rd(0, 1), qa = rd(0, 0);
#pragma unroll
        for (int t = 0; t < NDT; ++t) {
          vec8 doa_n = doa, qa_n = qa;
          if (t + 1 < NDT) {
            doa_n = rd(t + 1, 1);
            qa_n = rd(t + 1, 0);
          }
          dvacc[t] = Elem<T>::mfma16(doa, pb, dvacc[t]);
          dkacc[t] = Elem<T>::mfma16(qa, dsb, dkacc[t]);
          doa = doa_n;
          qa = qa_n;
          __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_sched_barrier(0);
      } else if constexpr (C::NT >= 256) {
        // head_dim 256: registers for one operand ahead only (dO^T of tile t, Q^T of tile t, dO^T of t + 1, ...);
        // without it every product waited for operands requested right before it
        vec8 cur = rd(0, 1);
#pragma unroll
        for (int i = 0; i < 2 * NDT; ++i) {
          vec8 nxt = cur;
          if (i + 1 < 2 * NDT) nxt = rd((i + 1) / 2, (i + 1) % 2 == 0 ? 1 : 0);
          if (i % 2 == 0) dvacc[i / 2] = Elem<T>::mfma16(cur, pb, dvacc[i / 2]);
          else dkacc[i / 2] = Elem<T>::mfma16(cur, dsb, dkacc[i / 2]);
          cur = nxt;
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
        for (int t = 0; t < NDT; ++t) {
          vec8 doa = rd(t, 1);
          dvacc[t] = Elem<T>::mfma16(doa, pb, dvacc[t]);
          vec8 qa = rd(t, 0);
          dkacc[t] = Elem<T>::mfma16(qa, dsb, dkacc[t]);
        }
      }
    }
    if (FUSE_DQ) {
      __syncthreads();  // dS^T of all waves is in LDS
      // dQ^T[d][row] = sum over the block's keys of K^T[d][key] dS^T[key][row]; row tiles are
      // dealt round-robin to the waves, both operands come from transposing LDS reads
      T* dqpart = reinterpret_cast<T*>(p.dq_part);
      const int64_t prow0 = ((int64_t)h * p.cap + start) * p.g;
      const int str_off = (4 * kg + (l16 >> 2)) * C::DSS + 4 * (l16 & 3);  // + 32*u*DSS + 16*rt
      const int tg = wv / C::RW;                     // which share of the d tiles
      constexpr int NTW = NDT / C::TG;               // d tiles per wave
      for (int rt = wv % C::RW; rt < NRT; rt += C::RW) {
        vec8 dsb[BK / 32];
#pragma unroll
        for (int u = 0; u < BK / 32; ++u)
          dsb[u] = lds_read_tr8<T>(&dSs[32 * u * C::DSS + str_off + 16 * rt], 16 * C::DSS);
        // the K copy is swizzled like the Q tile (same row pattern)
        auto kread = [&](int tt, int u) {
          return lds_read_tr8<T>(lds_ptr<T>(tr_addr0 ^ (32u * (tg * NTW + tt))) + (K_BYTES / 2 + 32 * u * C::KS), 16 * C::KS);
        };
        auto put = [&](int tt, const f32x4& acc) {
          vec4 x;
#pragma unroll
          for (int i = 0; i < 4; ++i) x[i] = (T)acc[i];
          if (C::STAGE_DQ) {
            store8(&dQst[l16 * C::DQS + 16 * tt + 4 * kg], x);
          } else {  // LDS too small for the staging tiles: direct 8-byte stores
            const int r = base + rt * 16 + l16;
            if (r < row_hi) store8(dqpart + (prow0 + r) * D + 16 * (tg * NTW + tt) + 4 * kg, x);
          }
        };
        if constexpr (D <= 128 && NTW % 2 == 0) {
          // two d tiles at a time (two independent accumulator chains), the K^T operands of the next two requested
          // before the products of the current two are issued
          constexpr int NKU = BK / 32;
          vec8 ka[2][NKU];
#pragma unroll
          for (int u = 0; u < NKU; ++u) {
            ka[0][u] = kread(0, u);
            ka[1][u] = kread(1, u);
          }
#pragma unroll
          for (int tt = 0; tt < NTW; tt += 2) {
            vec8 kn[2][NKU];
#pragma unroll
            for (int u = 0; u < NKU; ++u) {
              kn[0][u] = tt + 2 < NTW ? kread(tt + 2, u) : ka[0][u];
              kn[1][u] = tt + 2 < NTW ? kread(tt + 3, u) : ka[1][u];
            }
            f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < NKU; ++u) {
              a0 = Elem<T>::mfma16(ka[0][u], dsb[u], a0);
              a1 = Elem<T>::mfma16(ka[1][u], dsb[u], a1);
            }
            put(tt, a0);
            put(tt + 1, a1);
#pragma unroll
            for (int u = 0; u < NKU; ++u) {
              ka[0][u] = kn[0][u];
              ka[1][u] = kn[1][u];
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        } else if constexpr (NTW % 2 == 0) {  // head_dim 256: pairs of d tiles, no operands held ahead
#pragma unroll
          for (int tt = 0; tt < NTW; tt += 2) {
            f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < BK / 32; ++u) {
              a0 = Elem<T>::mfma16(kread(tt, u), dsb[u], a0);
              a1 = Elem<T>::mfma16(kread(tt + 1, u), dsb[u], a1);
            }
            put(tt, a0);
            put(tt + 1, a1);
          }
        } else {
#pragma unroll
          for (int tt = 0; tt < NTW; ++tt) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < BK / 32; ++u) acc = Elem<T>::mfma16(kread(tt, u), dsb[u], acc);
            put(tt, acc);
          }
        }
        // [16 rows][DW] piece -> row-coalesced 16-byte stores (CPW lanes per row)
        __builtin_amdgcn_wave_barrier();
        constexpr int CPW = C::DW / 8, RPI = 64 / CPW;
        if constexpr (C::STAGE_DQ) {  // all pieces read from the staging tile first, then stored
          vec8 xs[16 / RPI];
#pragma unroll
          for (int j = 0; j < 16 / RPI; ++j) xs[j] = load16<vec8>(&dQst[(lane / CPW + RPI * j) * C::DQS + (lane % CPW) * 8]);
#pragma unroll
          for (int j = 0; j < 16 / RPI; ++j) {
            const int r = base + rt * 16 + lane / CPW + RPI * j;
            if (r < row_hi) store16_stream(dqpart + (prow0 + r) * D + tg * C::DW + (lane % CPW) * 8, xs[j]);
          }
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
    if (FUSE_DQ) __builtin_amdgcn_s_setprio(0);
    // With the fused dQ every wave has passed the barrier above after its last read of the Q / dO tiles (the dQ
    // products read the dS^T tile and the K copy only): the rows of the next pass go into LDS without another
    // barrier in front, and one barrier ends the pass.
    if (!FUSE_DQ) __syncthreads();
    if (more) stash();
    __syncthreads();
  }

  // accumulators: dV^T[d = 16*t + 4*kg + i][key]
  if (ntile_b == 1) {
    if (key_ok) {
      T* dkrow = reinterpret_cast<T*>(p.dk) + (int64_t)ktok * p.dk_sn + (int64_t)h * p.dk_sh + 4 * kg;
      T* dvrow = reinterpret_cast<T*>(p.dv) + (int64_t)ktok * p.dk_sn + (int64_t)h * p.dk_sh + 4 * kg;
#pragma unroll
      for (int t = 0; t < NDT; ++t) {
        vec4 a, b;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a[i] = (T)dkacc[t][i];
          b[i] = (T)dvacc[t][i];
        }
        store8(dkrow + 16 * t, a);
        store8(dvrow + 16 * t, b);
      }
    }
  } else {
    float* part = p.dkdv_part + ((int64_t)h * p.max_tiles + w) * (2 * BK * D) + key * D + 4 * kg;
#pragma unroll
    for (int t = 0; t < NDT; ++t) {
      __builtin_nontemporal_store(dkacc[t], reinterpret_cast<f32x4*>(part + 16 * t));
      __builtin_nontemporal_store(dvacc[t], reinterpret_cast<f32x4*>(part + BK * D + 16 * t));
    }
  }
}

// Blocks with no selecting query get zeros; blocks split over several
// work-groups get the fixed-order sum of their fp32 partials.
// (bx, h, bz) of n_z: the position of the work-group in the grid of attn_bwd_dkdv_reduce_kernel; UB partial loads
// are issued together
template <typename T, int D, int BK, int MODE, int UB>
__device__ __forceinline__ void dkdv_reduce_block(const SelBwdParams& p, int bx, int h, int bz, int n_z) {
  typedef typename Elem<T>::vec4 vec4;
  const int32_t* tp = p.tile_prefix + h * (p.max_blocks + 1);
  const int n_blocks = p.cu_blocks[p.batch];
  // a work-group looks at KV_REDUCE_SPAN blocks at once: almost all of them have a single tile, whose
  // work-group wrote dK / dV itself
  __shared__ int todo[KV_REDUCE_SPAN];
  __shared__ int n_todo;
  const int gb0 = bx * KV_REDUCE_SPAN;
  if (threadIdx.x < WAVE) {
    static_assert(KV_REDUCE_SPAN == WAVE, "one lane per block of the span");
    const int gbi = gb0 + threadIdx.x;
    const bool multi = gbi < n_blocks && tp[gbi + 1] - tp[gbi] != 1;  // no tile at all: zeros
    const uint64_t m = __ballot(multi);
    if (multi) todo[__popcll(m & ((1ull << threadIdx.x) - 1))] = gbi;
    if (threadIdx.x == 0) n_todo = __popcll(m);
  }
  __syncthreads();
  // unit of work: 256 consecutive (key, 4 dims) items of one block; the gridDim.z work-groups of the span
  // take the units round-robin
  constexpr int CH = BK * (D / 4) / 256;
  for (int u_ = bz; u_ < n_todo * CH; u_ += n_z) {
    const int gb = todo[u_ / CH];
    const int t0 = tp[gb], nt = tp[gb + 1] - t0;
    KvBlock<MODE, BK> blk;
    blk.init(p, gb);
    {
      const int c = (u_ % CH) * 256 + threadIdx.x;
      const int key = c / (D / 4), d4 = (c % (D / 4)) * 4;
      const int tok = blk.key_row0 + key;
      if (key >= blk.n_keys_valid) continue;
      f32x4 sk = {0.f, 0.f, 0.f, 0.f}, sv = {0.f, 0.f, 0.f, 0.f};
      const float* part0 = p.dkdv_part + ((int64_t)h * p.max_tiles + t0) * (2 * BK * D) + key * D + d4;
      // the loads of a batch are issued together (one memory latency per batch), the adds keep the tile order
      for (int tb = 0; tb < nt; tb += UB) {
        f32x4 xk[UB], xv[UB];
#pragma unroll
        for (int u = 0; u < UB; ++u) {
          const float* part = part0 + (int64_t)max(min(tb + u, nt - 1), 0) * (2 * BK * D);
          xk[u] = *reinterpret_cast<const f32x4*>(part);
          xv[u] = *reinterpret_cast<const f32x4*>(part + BK * D);
        }
#pragma unroll
        for (int u = 0; u < UB; ++u)
          if (tb + u < nt) {
            sk += xk[u];
            sv += xv[u];
          }
      }
      vec4 a, b;
#pragma unroll
      for (int i2 = 0; i2 < 4; ++i2) {
        a[i2] = (T)sk[i2];
        b[i2] = (T)sv[i2];
      }
      store8(reinterpret_cast<T*>(p.dk) + (int64_t)tok * p.dk_sn + (int64_t)h * p.dk_sh + d4, a);
      store8(reinterpret_cast<T*>(p.dv) + (int64_t)tok * p.dk_sn + (int64_t)h * p.dk_sh + d4, b);
    }
  }
}

template <typename T, int D, int BK, int MODE>
__global__ void __launch_bounds__(256)
attn_bwd_dkdv_reduce_kernel(SelBwdParams p) {
  dkdv_reduce_block<T, D, BK, MODE, 8>(p, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.z);
}


}  // namespace fsa
