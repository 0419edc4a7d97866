// Inverted block->query index for selected attention (gfx950).
//
// The (query, slot) entries of topk_idx are keyed by global block id and put
// through a stable LSD radix sort (8-bit digits, wave64 ballot ranking), so
// that inside every block the queries appear in ascending order - the order the
// reference obtains by compacting a dense [nblk, N] table
// (fsa/ops/FSA_topk_sparse_attention.py:1016).  Work and memory are linear in
// N*T; nothing of size nblk*N is ever materialised.
#include "fsa_common.h"

#include <stdlib.h>

namespace fsa {

constexpr int RS_THREADS = 256;
constexpr int RS_WAVES = RS_THREADS / WAVE;
constexpr int RS_ROUNDS = 8;
constexpr int RS_PER_WAVE = RS_ROUNDS * WAVE;   // 512 consecutive items per wave
constexpr int RS_TILE = RS_WAVES * RS_PER_WAVE; // 2048 items per work-group
constexpr int SCAN_THREADS = 1024;

// Exclusive scan of one int per thread over a SCAN_THREADS-wide block.
__device__ __forceinline__ int block_exclusive_scan(int v, int* total) {
  __shared__ int wave_sums[SCAN_THREADS / WAVE];
  __shared__ int block_total;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  int inc = v;
#pragma unroll
  for (int o = 1; o < WAVE; o <<= 1) {
    int t = __shfl_up(inc, o, WAVE);
    if (lane >= o) inc += t;
  }
  if (lane == WAVE - 1) wave_sums[w] = inc;
  __syncthreads();
  if (w == 0) {
    int s = lane < (int)(blockDim.x / WAVE) ? wave_sums[lane] : 0;
    int si = s;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
      int t = __shfl_up(si, o, WAVE);
      if (lane >= o) si += t;
    }
    if (lane < (int)(blockDim.x / WAVE)) wave_sums[lane] = si - s;
    if (lane == WAVE - 1) block_total = si;
  }
  __syncthreads();
  int r = wave_sums[w] + inc - v;
  *total = block_total;
  __syncthreads();
  return r;
}

__global__ void cu_blocks_kernel(const int32_t* __restrict__ cu_seqlens, int batch, int block_size,
                                 int32_t* __restrict__ cu_blocks) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int acc = 0;
    cu_blocks[0] = 0;
    for (int s = 0; s < batch; ++s) {
      int len = cu_seqlens[s + 1] - cu_seqlens[s];
      acc += (len + block_size - 1) / block_size;
      cu_blocks[s + 1] = acc;
    }
  }
}

// key = global block id, or `sentinel` for padding / out-of-range ids; val = n*T + t
__global__ void __launch_bounds__(256)
make_keys_kernel(const int32_t* __restrict__ topk_idx, int64_t stride_h, int64_t stride_n,
                 const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ cu_blocks,
                 int batch, int64_t n_items, int topk, uint32_t sentinel,
                 uint32_t* __restrict__ keys, uint32_t* __restrict__ vals) {
  const int h = blockIdx.y;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n_items) return;
  const int token = (int)(idx / topk);
  const int t = (int)(idx - (int64_t)token * topk);
  const int b = topk_idx[h * stride_h + (int64_t)token * stride_n + t];
  const int s = upper_seg(cu_seqlens, batch, token);
  const int b0 = cu_blocks[s], nb = cu_blocks[s + 1] - b0;
  keys[h * n_items + idx] = (b >= 0 && b < nb) ? (uint32_t)(b0 + b) : sentinel;
  vals[h * n_items + idx] = (uint32_t)idx;
}

// table[h][digit][tile] = number of items of the tile with that digit
__global__ void __launch_bounds__(RS_THREADS)
radix_hist_kernel(const uint32_t* __restrict__ keys, int64_t n_items, int shift, int ntiles,
                  uint32_t* __restrict__ table) {
  __shared__ uint32_t hist[256];
  const int h = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;
  hist[tid] = 0;
  __syncthreads();
  const uint32_t* kh = keys + h * n_items;
#pragma unroll
  for (int j = 0; j < RS_ROUNDS; ++j) {
    int64_t idx = (int64_t)tile * RS_TILE + j * RS_THREADS + tid;
    if (idx < n_items) atomicAdd(&hist[(kh[idx] >> shift) & 255u], 1u);
  }
  __syncthreads();
  table[((int64_t)h * 256 + tid) * ntiles + tile] = hist[tid];
}

// Per (head, digit) row: in-place exclusive scan over the tiles; the row total
// goes to totals[h][digit] (the scatter kernel scans those 256 values itself).
__global__ void __launch_bounds__(256)
radix_scan_kernel(uint32_t* __restrict__ table, int ntiles, uint32_t* __restrict__ totals) {
  const int d = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  uint32_t* row = table + ((int64_t)h * 256 + d) * ntiles;
  int carry = 0;
  for (int base = 0; base < ntiles; base += 256) {
    const int i = base + tid;
    const int v = i < ntiles ? (int)row[i] : 0;
    int total;
    const int ex = block_exclusive_scan(v, &total);
    if (i < ntiles) row[i] = (uint32_t)(carry + ex);
    carry += total;
  }
  if (tid == 0) totals[h * 256 + d] = (uint32_t)carry;
}

// Stable scatter of one 8-bit digit.  Item order inside a tile is
// (wave, round, lane), i.e. the original order.
__global__ void __launch_bounds__(RS_THREADS)
radix_scatter_kernel(const uint32_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in,
                     uint32_t* __restrict__ keys_out, uint32_t* __restrict__ vals_out,
                     int64_t n_items, int shift, int ntiles, const uint32_t* __restrict__ table,
                     const uint32_t* __restrict__ totals) {
  __shared__ uint32_t cnt[RS_WAVES][256];
  const int h = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & (WAVE - 1), w = tid / WAVE;
  for (int i = tid; i < RS_WAVES * 256; i += RS_THREADS) (&cnt[0][0])[i] = 0;
  __syncthreads();
  const uint32_t* kh = keys_in + h * n_items;
  const uint32_t* vh = vals_in + h * n_items;
  uint32_t key[RS_ROUNDS], val[RS_ROUNDS], rank[RS_ROUNDS];
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int r = 0; r < RS_ROUNDS; ++r) {
    const int64_t idx = (int64_t)tile * RS_TILE + w * RS_PER_WAVE + r * WAVE + lane;
    const bool ok = idx < n_items;
    key[r] = ok ? kh[idx] : 0u;
    val[r] = ok ? vh[idx] : 0u;
    const uint32_t d = (key[r] >> shift) & 255u;
    uint64_t peers = __ballot(ok);
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
      const bool one = (d >> bit) & 1u;
      const uint64_t b = __ballot(one);
      peers &= one ? b : ~b;
    }
    uint32_t old = 0;
    if (ok) {
      old = cnt[w][d];
      rank[r] = old + (uint32_t)__popcll(peers & lt_mask);
    } else {
      rank[r] = 0;
    }
    __builtin_amdgcn_wave_barrier();
    if (ok && (peers & lt_mask) == 0) cnt[w][d] = old + (uint32_t)__popcll(peers);
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();
  int all_items;
  const int digit_base = block_exclusive_scan((int)totals[h * 256 + tid], &all_items);
  {  // per digit: global base of this tile + exclusive prefix over waves
    const int d = tid;
    uint32_t run = (uint32_t)digit_base + table[((int64_t)h * 256 + d) * ntiles + tile];
#pragma unroll
    for (int ww = 0; ww < RS_WAVES; ++ww) {
      uint32_t c = cnt[ww][d];
      cnt[ww][d] = run;
      run += c;
    }
  }
  __syncthreads();
  uint32_t* ko = keys_out + h * n_items;
  uint32_t* vo = vals_out + h * n_items;
#pragma unroll
  for (int r = 0; r < RS_ROUNDS; ++r) {
    const int64_t idx = (int64_t)tile * RS_TILE + w * RS_PER_WAVE + r * WAVE + lane;
    if (idx < n_items) {
      const uint32_t d = (key[r] >> shift) & 255u;
      const uint32_t dst = cnt[w][d] + rank[r];
      ko[dst] = key[r];
      vo[dst] = val[r];
    }
  }
}

__global__ void __launch_bounds__(256)
finalize_items_kernel(const uint32_t* __restrict__ keys, const uint32_t* __restrict__ vals,
                      int64_t n_items, int topk, uint32_t sentinel,
                      int32_t* __restrict__ sel_tokens, int32_t* __restrict__ slot_of) {
  const int h = blockIdx.y;
  const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (p >= n_items) return;
  const uint32_t key = keys[h * n_items + p];
  const uint32_t val = vals[h * n_items + p];
  const bool ok = key != sentinel;
  sel_tokens[h * n_items + p] = ok ? (int32_t)(val / (uint32_t)topk) : -1;
  slot_of[h * n_items + val] = ok ? (int32_t)p : -1;
}

// starts[h][gb] = first position whose key >= gb; counts = adjacent difference
__global__ void __launch_bounds__(256)
starts_kernel(const uint32_t* __restrict__ keys, int64_t n_items, int64_t max_blocks,
              int32_t* __restrict__ starts, int32_t* __restrict__ counts) {
  const int h = blockIdx.y;
  const int64_t gb = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (gb > max_blocks) return;
  const uint32_t* kh = keys + h * n_items;
  auto lower = [&](uint32_t x) {
    int64_t lo = 0, hi = n_items;
    while (lo < hi) {
      int64_t mid = (lo + hi) >> 1;
      if (kh[mid] < x) lo = mid + 1; else hi = mid;
    }
    return (int32_t)lo;
  };
  const int32_t s0 = lower((uint32_t)gb);
  starts[h * (max_blocks + 1) + gb] = s0;
  if (gb < max_blocks) counts[h * max_blocks + gb] = lower((uint32_t)gb + 1) - s0;
}

// ------------------------------------------------------------------------------------------------
// Counting path (a few thousand blocks at most): one pass that counts, per tile of consecutive queries,
// the entries of every block, a scan of those counts over the tiles, and one pass that places every entry:
// position = start of its block + entries of the block in earlier tiles + earlier entries of the block inside
// the tile.  Entries are visited in (query, slot) order, so every block's list is ascending in the query id.
// Padding entries form one extra "block" (id max_blocks) behind all others: the -1 tail of sel_tokens.
constexpr int CT_THREADS = 256;
constexpr int CT_WAVES = CT_THREADS / WAVE;
constexpr int CT_ITEMS = 4096;                       // entries per tile (a whole number of queries)
constexpr int CT_ROUNDS = CT_ITEMS / CT_THREADS;     // entries per thread
constexpr int CT_MAX_BUCKETS = 4096;                 // max_blocks + 1 must not exceed this (LDS: 16 B per bucket)

// Sequences that the consecutive queries of a tile belong to.  Almost every tile lies inside one sequence: its
// block range is then looked up once per work-group, and the bucket of an entry is its block id plus a constant -
// the loads of all entries of a thread are independent and in flight together.  (A search per entry puts a chain of
// dependent loads into every round.)
struct SeqSpan {
  int s_lo, s_hi;  // sequence of the first / last query
  int b0, nb;      // first global block and block count of sequence s_lo
};
__device__ __forceinline__ SeqSpan seq_span(const int32_t* __restrict__ cu_seqlens,
                                            const int32_t* __restrict__ cu_blocks, int batch, int tok_first,
                                            int tok_last) {
  SeqSpan sp;
  sp.s_lo = upper_seg(cu_seqlens, batch, tok_first);
  sp.s_hi = upper_seg(cu_seqlens, batch, tok_last);
  sp.b0 = cu_blocks[sp.s_lo];
  sp.nb = cu_blocks[sp.s_lo + 1] - sp.b0;
  return sp;
}

// i / d for 0 <= i < 2^22, d >= 1 with rcp = 1.0f / d: the float product is off by less than one, one correction
// step makes it exact (a handful of instructions against some forty for the integer division)
__device__ __forceinline__ int div_small(int i, int d, float rcp) {
  int q = (int)((float)i * rcp);
  const int r = i - q * d;
  q += (r >= d ? 1 : 0) - (r < 0 ? 1 : 0);
  return q;
}

// Block ids of CT_ROUNDS entries of a tile: entry numbers idx[r] (negative: none).  All loads are issued together,
// without branches, and before anything that waits for another load.
__device__ __forceinline__ void load_block_ids(const int32_t* __restrict__ topk_idx, int64_t stride_h,
                                               int64_t stride_n, int h, int tok0, int topk, int n_it,
                                               const int* idx, int* raw) {
  const float rcp = 1.0f / (float)topk;
  const int32_t* base = topk_idx + h * stride_h;
#pragma unroll
  for (int r = 0; r < CT_ROUNDS; ++r) {
    const int i = min(max(idx[r], 0), n_it - 1);
    const int qi = div_small(i, topk, rcp), t = i - qi * topk;
    raw[r] = base[(int64_t)(tok0 + qi) * stride_n + t];
  }
}

// block ids -> buckets (global block ids; `sentinel` for padding and out-of-range ids; -1 where there is no entry)
__device__ __forceinline__ void ids_to_buckets(const int32_t* __restrict__ cu_seqlens,
                                               const int32_t* __restrict__ cu_blocks, int batch, const SeqSpan& sp,
                                               int tok0, int topk, int sentinel, const int* idx, const int* raw,
                                               int* key) {
  if (sp.s_lo == sp.s_hi) {  // uniform over the work-group
#pragma unroll
    for (int r = 0; r < CT_ROUNDS; ++r) {
      const int b = raw[r];
      key[r] = idx[r] < 0 ? -1 : (b >= 0 && b < sp.nb) ? sp.b0 + b : sentinel;
    }
  } else {
    const float rcp = 1.0f / (float)topk;
#pragma unroll
    for (int r = 0; r < CT_ROUNDS; ++r) {
      const int b = raw[r];  // raw and key may be the same array
      int k = -1;
      if (idx[r] >= 0) {
        const int s = upper_seg(cu_seqlens, batch, tok0 + div_small(idx[r], topk, rcp));
        const int b0 = cu_blocks[s], nb = cu_blocks[s + 1] - b0;
        k = (b >= 0 && b < nb) ? b0 + b : sentinel;
      }
      key[r] = k;
    }
  }
}

// table[h][tile][bucket] = entries of the tile that fall into the bucket (a tile writes one contiguous row)
__global__ void __launch_bounds__(CT_THREADS)
count_tiles_kernel(const int32_t* __restrict__ topk_idx, int64_t stride_h, int64_t stride_n,
                   const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ cu_blocks, int batch,
                   int64_t n_tokens, int topk, int q_per_tile, int ntiles, int nbuckets,
                   int32_t* __restrict__ table) {
  extern __shared__ int hist[];
  const int h = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;
  const int64_t tok0 = (int64_t)tile * q_per_tile;
  const int n_q = (int)min((int64_t)q_per_tile, n_tokens - tok0);
  int key[CT_ROUNDS], idx[CT_ROUNDS];  // the tile has at most CT_ITEMS entries (host check)
#pragma unroll
  for (int r = 0; r < CT_ROUNDS; ++r) {
    const int i = tid + r * CT_THREADS;
    idx[r] = i < n_q * topk ? i : -1;
  }
  load_block_ids(topk_idx, stride_h, stride_n, h, (int)tok0, topk, n_q * topk, idx, key);
  for (int b = tid; b < nbuckets; b += CT_THREADS) hist[b] = 0;   // while the ids are on their way
  __syncthreads();
  const SeqSpan sp = seq_span(cu_seqlens, cu_blocks, batch, (int)tok0, (int)tok0 + n_q - 1);
  ids_to_buckets(cu_seqlens, cu_blocks, batch, sp, (int)tok0, topk, nbuckets - 1, idx, key, key);
#pragma unroll
  for (int r = 0; r < CT_ROUNDS; ++r)
    if (key[r] >= 0) atomicAdd(&hist[key[r]], 1);
  __syncthreads();
  for (int b = tid; b < nbuckets; b += CT_THREADS) table[((int64_t)h * ntiles + tile) * nbuckets + b] = hist[b];
}

// Exclusive scan of the table over the tiles, bucket by bucket; the total of a bucket is its entry count.  A
// work-group takes 64 buckets (one per lane: the reads of a tile row are contiguous) and each of its waves an equal
// share of the tiles: column sums of the shares, then the running prefix written back over the counts.
constexpr int ST_WAVES = 16;
__global__ void __launch_bounds__(ST_WAVES * WAVE)
scan_tiles_kernel(int32_t* __restrict__ table, int ntiles, int nbuckets, int64_t max_blocks,
                  int32_t* __restrict__ counts, int32_t* __restrict__ bucket_total) {
  __shared__ int part[ST_WAVES][WAVE];
  const int h = blockIdx.y, lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  const int b = blockIdx.x * WAVE + lane;
  const bool live = b < nbuckets;
  const int per = (ntiles + ST_WAVES - 1) / ST_WAVES;
  const int t0 = min(ntiles, w * per), t1 = min(ntiles, t0 + per);
  int32_t* col = table + (int64_t)h * ntiles * nbuckets + (live ? b : 0);
  int sum = 0;
  if (live) {
#pragma unroll 8
    for (int t = t0; t < t1; ++t) sum += col[(int64_t)t * nbuckets];
  }
  part[w][lane] = sum;
  __syncthreads();
  int run = 0;
  for (int ww = 0; ww < w; ++ww) run += part[ww][lane];
  if (live) {
#pragma unroll 8
    for (int t = t0; t < t1; ++t) {
      const int v = col[(int64_t)t * nbuckets];
      col[(int64_t)t * nbuckets] = run;
      run += v;
    }
    if (w == ST_WAVES - 1) {  // the last share ends at the total
      bucket_total[h * nbuckets + b] = run;
      if (b < max_blocks) counts[h * max_blocks + b] = run;
    }
  }
}

// Exclusive scans of two ints per thread over the CT_THREADS of a work-group.
__device__ __forceinline__ void block_exclusive_scan2(int a, int b, int* ea, int* eb) {
  __shared__ int wa[CT_WAVES], wb[CT_WAVES];
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  int ia = a, ib = b;
#pragma unroll
  for (int o = 1; o < WAVE; o <<= 1) {
    const int ta = __shfl_up(ia, o, WAVE), tb = __shfl_up(ib, o, WAVE);
    if (lane >= o) {
      ia += ta;
      ib += tb;
    }
  }
  if (lane == WAVE - 1) {
    wa[w] = ia;
    wb[w] = ib;
  }
  __syncthreads();
  int offa = 0, offb = 0;
  for (int ww = 0; ww < w; ++ww) {
    offa += wa[ww];
    offb += wb[ww];
  }
  *ea = offa + ia - a;
  *eb = offb + ib - b;
  __syncthreads();
}

// LDS of place_items_kernel in ints: per-wave counters [CT_WAVES][nbuckets], reused as the list of positions of the
// tile's sorted entries [CT_ITEMS]; per-bucket offset [nbuckets]; entry numbers of the sorted entries [CT_ITEMS] as
// 16-bit values
__host__ __device__ inline int place_lds_ints(int nbuckets) {
  const int a = CT_WAVES * nbuckets > CT_ITEMS ? CT_WAVES * nbuckets : CT_ITEMS;
  return a + nbuckets + CT_ITEMS / 2;
}

// Places the entries of one tile.  Position of an entry = start of its bucket (exclusive scan of the bucket totals,
// done here by every work-group; tile 0 also stores it as `starts`) + entries of the bucket in earlier tiles (table)
// + earlier entries of the bucket inside the tile.  The tile's entries are first put into bucket order in LDS, so
// that neighbouring lanes store to neighbouring positions of `sel_tokens` (the few entries that a tile has in one
// bucket are one store transaction instead of one each).
// KEY_BITS: bits of a bucket id that the lanes of a wave are matched on (2^KEY_BITS >= nbuckets); a constant, so
// that the matching below is straight-line code - as a loop over a run-time count it spends as much on the loop as
// on the ballots.
template <int KEY_BITS>
__global__ void __launch_bounds__(CT_THREADS)
place_items_kernel(const int32_t* __restrict__ topk_idx, int64_t stride_h, int64_t stride_n,
                   const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ cu_blocks, int batch,
                   int64_t n_tokens, int topk, int q_per_tile, int ntiles, int nbuckets,
                   const int32_t* __restrict__ table, const int32_t* __restrict__ bucket_total,
                   int32_t* __restrict__ starts, int32_t* __restrict__ sel_tokens, int32_t* __restrict__ slot_of) {
  extern __shared__ int lds[];
  int* cnt = lds;                                  // [CT_WAVES][nbuckets]
  int* sorted_pos = lds;                           // [CT_ITEMS], once the counters are no longer needed
  int* delta = lds + max(CT_WAVES * nbuckets, CT_ITEMS);   // [nbuckets]: position in sel_tokens - position in the tile
  uint16_t* sorted_item = reinterpret_cast<uint16_t*>(delta + nbuckets);  // [CT_ITEMS]
  __shared__ int n_real_s;
  // Work-groups go to the eight XCDs in turn, and each XCD has its own L2.  Consecutive tiles append to the same
  // lines of sel_tokens: tiles are dealt so that an XCD gets a contiguous eighth of them (gridDim.x is a multiple
  // of eight), and the pieces of a line meet in one L2 instead of leaving eight of them as partial lines.
  const int h = blockIdx.y, tid = threadIdx.x;
  const int tile = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (tile >= ntiles) return;
  const int lane = tid & (WAVE - 1), w = tid / WAVE;
  const int64_t tok0 = (int64_t)tile * q_per_tile;
  const int n_q = (int)min((int64_t)q_per_tile, n_tokens - tok0);
  const int n_it = n_q * topk;
  // wave w owns entries [w * per_wave, (w + 1) * per_wave) of the tile, 64 per round, in order
  const int per_wave = (q_per_tile * topk + CT_WAVES - 1) / CT_WAVES;
  const int rounds = (per_wave + WAVE - 1) / WAVE;   // <= CT_ROUNDS (host check)
  int key[CT_ROUNDS], rank[CT_ROUNDS];
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  int* my_cnt = cnt + w * nbuckets;
  // all bucket ids first (the loads of every round in flight together), then the ordered ranking
  {
    int idx[CT_ROUNDS];
#pragma unroll
    for (int r = 0; r < CT_ROUNDS; ++r) {
      const int i = w * per_wave + r * WAVE + lane;
      idx[r] = (r < rounds && r * WAVE + lane < per_wave && i < n_it) ? i : -1;
      rank[r] = 0;
    }
    load_block_ids(topk_idx, stride_h, stride_n, h, (int)tok0, topk, n_it, idx, key);
    for (int i = tid; i < CT_WAVES * nbuckets; i += CT_THREADS) cnt[i] = 0;   // while the ids are on their way
    __syncthreads();
    const SeqSpan sp = seq_span(cu_seqlens, cu_blocks, batch, (int)tok0, (int)tok0 + n_q - 1);
    ids_to_buckets(cu_seqlens, cu_blocks, batch, sp, (int)tok0, topk, nbuckets - 1, idx, key, key);
  }
#pragma unroll
  for (int r = 0; r < CT_ROUNDS; ++r) {
    if (r < rounds) {  // uniform
      const bool ok = key[r] >= 0;
      const int kb = ok ? key[r] : 0;
      const uint64_t valid = __ballot(ok);
      uint32_t p_lo = (uint32_t)valid, p_hi = (uint32_t)(valid >> 32);
#pragma unroll
      for (int bit = 0; bit < KEY_BITS; ++bit) {
        // lanes whose bit is set keep the lanes of the ballot, the others its complement: one sign-extending
        // bit-field extract gives the XOR mask (0 or ~0) and the predicate of the ballot
        const uint32_t flip = (uint32_t)__builtin_amdgcn_sbfe(~kb, bit, 1);
        const uint64_t bb = __ballot(flip == 0u);
        p_lo &= (uint32_t)bb ^ flip;
        p_hi &= (uint32_t)(bb >> 32) ^ flip;
      }
      const uint64_t peers = ((uint64_t)p_hi << 32) | p_lo;
      int old = 0;
      if (ok) {
        old = my_cnt[kb];
        rank[r] = old + __popcll(peers & lt_mask);
      }
      __builtin_amdgcn_wave_barrier();
      if (ok && (peers & lt_mask) == 0) my_cnt[kb] = old + __popcll(peers);
      __builtin_amdgcn_wave_barrier();
    }
  }
  __syncthreads();
  // Thread t finishes buckets [t * per, (t + 1) * per): two exclusive scans over the buckets - of the bucket totals
  // (start of the bucket in sel_tokens) and of the tile's own counts (start of the bucket in the sorted tile).
  constexpr int BPT = CT_MAX_BUCKETS / CT_THREADS;
  const int per = (nbuckets + CT_THREADS - 1) / CT_THREADS;   // <= BPT
  const int32_t* tot = bucket_total + h * nbuckets;
  const int32_t* trow = table + ((int64_t)h * ntiles + tile) * nbuckets;
  int tot_r[BPT], tab_r[BPT];
  int sum_tot = 0, sum_tile = 0;
#pragma unroll
  for (int j = 0; j < BPT; ++j) {
    const int b = tid * per + j;
    tot_r[j] = 0;
    tab_r[j] = 0;
    if (j < per && b < nbuckets) {
      tot_r[j] = tot[b];
      tab_r[j] = trow[b];
      sum_tot += tot_r[j];
#pragma unroll
      for (int ww = 0; ww < CT_WAVES; ++ww) sum_tile += cnt[ww * nbuckets + b];
    }
  }
  int g_run, l_run;
  block_exclusive_scan2(sum_tot, sum_tile, &g_run, &l_run);
#pragma unroll
  for (int j = 0; j < BPT; ++j) {
    const int b = tid * per + j;
    if (j < per && b < nbuckets) {
      if (tile == 0) starts[h * nbuckets + b] = g_run;   // [Hkv, max_blocks + 1] with nbuckets = max_blocks + 1
      delta[b] = g_run + tab_r[j] - l_run;
      if (b == nbuckets - 1) n_real_s = l_run;            // the padding bucket is the last one
#pragma unroll
      for (int ww = 0; ww < CT_WAVES; ++ww) {
        const int c = cnt[ww * nbuckets + b];
        cnt[ww * nbuckets + b] = l_run;
        l_run += c;
      }
      g_run += tot_r[j];
    }
  }
  __syncthreads();
  const int64_t n_items = n_tokens * topk;
  int32_t* st = sel_tokens + h * n_items;
  int32_t* so = slot_of + h * n_items;
  const int n_real = n_real_s;
  // position in the sorted tile (kept in key[]) and in sel_tokens (rank[]); slot_of in entry order
#pragma unroll
  for (int r = 0; r < CT_ROUNDS; ++r) {
    if (r < rounds && key[r] >= 0) {
      const int i = w * per_wave + r * WAVE + lane;
      const int lpos = my_cnt[key[r]] + rank[r];
      const int pos = lpos + delta[key[r]];
      so[tok0 * topk + i] = key[r] != nbuckets - 1 ? pos : -1;
      key[r] = lpos;
      rank[r] = pos;
    } else {
      key[r] = -1;
    }
  }
  __syncthreads();  // the counters are dead: their memory becomes the position list
#pragma unroll
  for (int r = 0; r < CT_ROUNDS; ++r) {
    if (key[r] >= 0) {
      sorted_pos[key[r]] = rank[r];
      sorted_item[key[r]] = (uint16_t)(w * per_wave + r * WAVE + lane);
    }
  }
  __syncthreads();
  const float rcp = 1.0f / (float)topk;
#pragma unroll
  for (int r = 0; r < CT_ROUNDS; ++r) {
    const int j = tid + r * CT_THREADS;
    if (j < n_it) st[sorted_pos[j]] = j < n_real ? (int32_t)(tok0 + div_small((int)sorted_item[j], topk, rcp)) : -1;
  }
}

// out[h, token, t * factor + j] = id of sub-block j of the selected block t, -1 if it lies after the query
__global__ void __launch_bounds__(256)
split_blocks_kernel(const int32_t* __restrict__ topk_idx, int64_t stride_h, int64_t stride_n,
                    const int32_t* __restrict__ cu_seqlens, int batch, int64_t n_out, int topk, int factor,
                    int sub_size, int32_t* __restrict__ out) {
  const int h = blockIdx.y;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n_out) return;
  const int per = topk * factor;
  const int token = (int)(idx / per);
  const int r = (int)(idx - (int64_t)token * per);
  const int t = r / factor, j = r - t * factor;
  const int b = topk_idx[h * stride_h + (int64_t)token * stride_n + t];
  const int s = upper_seg(cu_seqlens, batch, token);
  const int qpos = token - cu_seqlens[s];
  const int64_t sb = (int64_t)b * factor + j;
  out[h * n_out + idx] = (b >= 0 && sb * sub_size <= qpos) ? (int32_t)sb : -1;
}

__global__ void __launch_bounds__(SCAN_THREADS)
tiles_kernel(const int32_t* __restrict__ counts, int64_t max_blocks, int group_size, int rows_per_tile,
             int32_t* __restrict__ tile_prefix, int32_t* __restrict__ tile_block, int64_t max_tiles) {
  const int h = blockIdx.x;
  const int32_t* c = counts + h * max_blocks;
  int32_t* tp = tile_prefix + h * (max_blocks + 1);
  const int64_t per = (max_blocks + SCAN_THREADS - 1) / SCAN_THREADS;
  const int64_t lo = (int64_t)threadIdx.x * per;
  const int64_t hi = lo + per < max_blocks ? lo + per : max_blocks;
  auto ntile = [&](int64_t gb) {
    return (int)(((int64_t)c[gb] * group_size + rows_per_tile - 1) / rows_per_tile);
  };
  int sum = 0;
  for (int64_t i = lo; i < hi; ++i) sum += ntile(i);
  int total;
  int run = block_exclusive_scan(sum, &total);
  for (int64_t i = lo; i < hi; ++i) {
    tp[i] = run;
    const int nt = ntile(i);
    // tile -> block, so that a work-group finds its block with one load instead of a binary search through tp
    if (tile_block)
      for (int t = 0; t < nt; ++t) tile_block[h * max_tiles + run + t] = (int32_t)i;
    run += nt;
  }
  if (threadIdx.x == 0) tp[max_blocks] = total;
}

}  // namespace fsa

using namespace fsa;

static void index_ws_layout(int64_t n_items, int hkv, size_t* off_keys, size_t* off_vals,
                            size_t* off_table, size_t* off_totals, size_t* total) {
  const size_t buf = align_up((size_t)n_items * hkv * 4, 256);
  const int64_t ntiles = (n_items + RS_TILE - 1) / RS_TILE;
  off_keys[0] = 0;
  off_keys[1] = buf;
  off_vals[0] = 2 * buf;
  off_vals[1] = 3 * buf;
  *off_table = 4 * buf;
  *off_totals = *off_table + align_up((size_t)hkv * 256 * ntiles * 4, 256);
  *total = *off_totals + align_up((size_t)hkv * 256 * 4, 256);
}

// The counting path needs max_blocks + 1 buckets in LDS (16 bytes each), at most CT_ROUNDS entries per thread
// and a [Hkv, buckets, tiles] table of moderate size; everything else takes the radix sort.
struct CountPlan {
  bool use;
  int q_per_tile, ntiles, nbuckets;
  size_t off_table, off_totals, total;
};
static CountPlan count_plan(int64_t total_tokens, int topk, int hkv, int64_t max_blocks) {
  CountPlan c = {};
  if (max_blocks + 1 > CT_MAX_BUCKETS || topk > CT_ITEMS / 4) return c;
  c.q_per_tile = CT_ITEMS / topk;
  c.ntiles = (int)((total_tokens + c.q_per_tile - 1) / c.q_per_tile);
  c.nbuckets = (int)max_blocks + 1;
  const size_t entries = (size_t)hkv * c.nbuckets * c.ntiles;
  if (entries > ((size_t)1 << 24)) return c;
  c.use = getenv("FSA_INDEX_RADIX") == nullptr;  // the environment switch forces the general path (for tests)
  c.off_table = 0;
  c.off_totals = align_up(entries * 4, 256);
  c.total = c.off_totals + align_up((size_t)hkv * c.nbuckets * 4, 256);
  return c;
}

extern "C" size_t fsa_index_workspace_bytes(int64_t total_tokens, int32_t topk, int32_t num_kv_heads,
                                            int64_t max_blocks) {
  const CountPlan c = count_plan(total_tokens, topk, num_kv_heads, max_blocks);
  if (c.use) return c.total;
  size_t ok[2], ov[2], ot, ott, total;
  index_ws_layout(total_tokens * topk, num_kv_heads, ok, ov, &ot, &ott, &total);
  return total;
}

extern "C" int fsa_build_index(const int32_t* topk_idx, int64_t topk_stride_h, int64_t topk_stride_n,
                               const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens,
                               int32_t num_kv_heads, int32_t topk, int32_t block_size,
                               int64_t max_blocks, int32_t* cu_blocks, int32_t* counts,
                               int32_t* starts, int32_t* sel_tokens, int32_t* slot_of,
                               void* workspace, size_t workspace_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(topk_idx && cu_seqlens && cu_blocks && counts && starts && sel_tokens && slot_of,
                "fsa_build_index: null pointer");
  FSA_CHECK_ARG(batch >= 1 && total_tokens >= 1 && num_kv_heads >= 1 && topk >= 1,
                "fsa_build_index: batch, total_tokens, num_kv_heads and topk must be positive");
  FSA_CHECK_ARG(block_size >= 1, "fsa_build_index: block_size must be positive");
  FSA_CHECK_ARG(max_blocks >= 1 && max_blocks < (1 << 24),
                "fsa_build_index: max_blocks=%lld out of range", (long long)max_blocks);
  const int64_t n_items = total_tokens * topk;
  FSA_CHECK_ARG(n_items < ((int64_t)1 << 31), "fsa_build_index: total_tokens*topk must be < 2^31");
  const size_t need = fsa_index_workspace_bytes(total_tokens, topk, num_kv_heads, max_blocks);
  if (workspace == nullptr || workspace_bytes < need) {
    set_error("fsa_build_index: workspace too small (%zu < %zu)", workspace_bytes, need);
    return FSA_ERR_WORKSPACE;
  }
  char* ws = (char*)workspace;
  ProfScope ps_("index_build", stream);  // the whole pipeline of small kernels as one record
  cu_blocks_kernel<<<1, 64, 0, stream>>>(cu_seqlens, batch, block_size, cu_blocks);

  const CountPlan c = count_plan(total_tokens, topk, num_kv_heads, max_blocks);
  if (c.use) {
    int32_t* table = (int32_t*)(ws + c.off_table);
    int32_t* totals = (int32_t*)(ws + c.off_totals);
    int key_bits = 1;
    while ((1 << key_bits) < c.nbuckets) ++key_bits;
    dim3 g_tiles(c.ntiles, num_kv_heads);
    count_tiles_kernel<<<g_tiles, CT_THREADS, (size_t)c.nbuckets * 4, stream>>>(
        topk_idx, topk_stride_h, topk_stride_n, cu_seqlens, cu_blocks, batch, total_tokens, topk, c.q_per_tile,
        c.ntiles, c.nbuckets, table);
    scan_tiles_kernel<<<dim3((c.nbuckets + WAVE - 1) / WAVE, num_kv_heads), ST_WAVES * WAVE, 0, stream>>>(
        table, c.ntiles, c.nbuckets, max_blocks, counts, totals);
    const size_t lds = (size_t)place_lds_ints(c.nbuckets) * 4;
    dim3 g_place((c.ntiles + 7) / 8 * 8, num_kv_heads);
#define FSA_PLACE(KB)                                                                                            \
  {                                                                                                              \
    static bool attr_done = false;                                                                               \
    if (!attr_done && lds > 48 * 1024) {                                                                         \
      hipError_t e = hipFuncSetAttribute((const void*)place_items_kernel<KB>,                                    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize,                     \
                                         place_lds_ints(CT_MAX_BUCKETS) * 4);                                    \
      if (e != hipSuccess) {                                                                                     \
        set_error("hipFuncSetAttribute(place_items_kernel): %s", hipGetErrorString(e));                          \
        return (int)e;                                                                                           \
      }                                                                                                          \
      attr_done = true;                                                                                          \
    }                                                                                                            \
    place_items_kernel<KB><<<g_place, CT_THREADS, lds, stream>>>(                                                \
        topk_idx, topk_stride_h, topk_stride_n, cu_seqlens, cu_blocks, batch, total_tokens, topk, c.q_per_tile,  \
        c.ntiles, c.nbuckets, table, totals, starts, sel_tokens, slot_of);                                       \
  }
    if (key_bits <= 7) FSA_PLACE(7)
    else if (key_bits <= 9) FSA_PLACE(9)
    else if (key_bits <= 10) FSA_PLACE(10)
    else if (key_bits <= 11) FSA_PLACE(11)
    else FSA_PLACE(12)
#undef FSA_PLACE
    FSA_CHECK_LAUNCH("fsa_build_index");
    return 0;
  }

  size_t ok[2], ov[2], ot, ott, total;
  index_ws_layout(n_items, num_kv_heads, ok, ov, &ot, &ott, &total);
  uint32_t* keys[2] = {(uint32_t*)(ws + ok[0]), (uint32_t*)(ws + ok[1])};
  uint32_t* vals[2] = {(uint32_t*)(ws + ov[0]), (uint32_t*)(ws + ov[1])};
  uint32_t* table = (uint32_t*)(ws + ot);
  uint32_t* totals = (uint32_t*)(ws + ott);
  const int ntiles = (int)((n_items + RS_TILE - 1) / RS_TILE);
  const uint32_t sentinel = (uint32_t)max_blocks;

  dim3 g_items((unsigned)((n_items + 255) / 256), num_kv_heads);
  make_keys_kernel<<<g_items, 256, 0, stream>>>(topk_idx, topk_stride_h, topk_stride_n, cu_seqlens,
                                                cu_blocks, batch, n_items, topk, sentinel, keys[0],
                                                vals[0]);
  int bits = 1;
  while (((uint64_t)1 << bits) <= (uint64_t)sentinel) ++bits;
  const int passes = (bits + 7) / 8;
  int cur = 0;
  for (int p = 0; p < passes; ++p) {
    dim3 g_tiles(ntiles, num_kv_heads);
    radix_hist_kernel<<<g_tiles, RS_THREADS, 0, stream>>>(keys[cur], n_items, 8 * p, ntiles, table);
    radix_scan_kernel<<<dim3(256, num_kv_heads), 256, 0, stream>>>(table, ntiles, totals);
    radix_scatter_kernel<<<g_tiles, RS_THREADS, 0, stream>>>(keys[cur], vals[cur], keys[cur ^ 1],
                                                             vals[cur ^ 1], n_items, 8 * p, ntiles,
                                                             table, totals);
    cur ^= 1;
  }
  finalize_items_kernel<<<g_items, 256, 0, stream>>>(keys[cur], vals[cur], n_items, topk, sentinel,
                                                     sel_tokens, slot_of);
  dim3 g_blocks((unsigned)((max_blocks + 1 + 255) / 256), num_kv_heads);
  starts_kernel<<<g_blocks, 256, 0, stream>>>(keys[cur], n_items, max_blocks, starts, counts);
  FSA_CHECK_LAUNCH("fsa_build_index");
  return 0;
}

extern "C" int fsa_split_topk_blocks(const int32_t* topk_idx, int64_t topk_stride_h, int64_t topk_stride_n,
                                     const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens,
                                     int32_t num_kv_heads, int32_t topk, int32_t block_size, int32_t factor,
                                     int32_t* out, void* stream_) {
  FSA_CHECK_ARG(topk_idx && cu_seqlens && out, "fsa_split_topk_blocks: null pointer");
  FSA_CHECK_ARG(batch >= 1 && total_tokens >= 1 && num_kv_heads >= 1 && topk >= 1,
                "fsa_split_topk_blocks: batch, total_tokens, num_kv_heads and topk must be positive");
  FSA_CHECK_ARG(factor >= 1 && block_size >= factor && block_size % factor == 0,
                "fsa_split_topk_blocks: factor must divide block_size");
  const int64_t n_out = total_tokens * topk * factor;
  FSA_CHECK_ARG(n_out < ((int64_t)1 << 31), "fsa_split_topk_blocks: total_tokens*topk*factor must be < 2^31");
  dim3 grid((unsigned)((n_out + 255) / 256), num_kv_heads);
  split_blocks_kernel<<<grid, 256, 0, (hipStream_t)stream_>>>(topk_idx, topk_stride_h, topk_stride_n, cu_seqlens,
                                                             batch, n_out, topk, factor, block_size / factor, out);
  FSA_CHECK_LAUNCH("fsa_split_topk_blocks");
  return 0;
}

int fsa::build_tiles(const int32_t* counts, int num_kv_heads, int64_t max_blocks, int group_size,
                     int rows_per_tile, int32_t* tile_prefix, int32_t* tile_block, int64_t max_tiles,
                     hipStream_t stream) {
  FSA_CHECK_ARG(counts && tile_prefix, "fsa_build_tiles: null pointer");
  FSA_CHECK_ARG(num_kv_heads >= 1 && max_blocks >= 1 && group_size >= 1 && rows_per_tile >= 1,
                "fsa_build_tiles: sizes must be positive");
  tiles_kernel<<<num_kv_heads, SCAN_THREADS, 0, stream>>>(counts, max_blocks, group_size, rows_per_tile,
                                                          tile_prefix, tile_block, max_tiles);
  FSA_CHECK_LAUNCH("fsa_build_tiles");
  return 0;
}

extern "C" int fsa_build_tiles(const int32_t* counts, int32_t num_kv_heads, int64_t max_blocks,
                               int32_t group_size, int32_t rows_per_tile, int32_t* tile_prefix,
                               void* stream_) {
  return fsa::build_tiles(counts, num_kv_heads, max_blocks, group_size, rows_per_tile, tile_prefix, nullptr, 0,
                          (hipStream_t)stream_);
}

extern "C" int64_t fsa_max_tiles(int64_t total_tokens, int32_t topk, int32_t group_size,
                                 int32_t rows_per_tile, int64_t max_blocks) {
  return (total_tokens * topk * group_size + rows_per_tile - 1) / rows_per_tile + max_blocks;
}
