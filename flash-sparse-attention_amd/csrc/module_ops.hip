// Kernels the attention layer needs around the hot path (gfx950):
//   rope          : rotary embedding on packed sequences (forward, and its inverse
//                   rotation = backward), positions start + j*stride per sequence
//   lc_fwd        : linear compression y[n,h,:] = sum_k x[n*stride+k,h,:] W[h,k] (+ bias)
//                   as a strided-window GEMM: Y^T = W^T X^T on 32x32x16 MFMA, W tiles
//                   through LDS with transposing reads, X rows straight from memory
//   lc_dx / lc_dw : its backward without atomics: dX^T = sum_r W[h,k_r] dY[n_r]^T per
//                   token phase, and dW[h,k] = X_k^T dY with both operands read
//                   transposed from LDS tiles
//
// Semantics: nsa_ref/module/rope.py:64-134, nsa_ref/ops/linear_compress.py:28-131
// (forward), :135-292 (backward, fp32 atomics there), :474-502 (positional bias).
#include "fsa_common.h"

namespace fsa {

// ------------------------------------------------------------------- rope ----
// One wave per token.  d/16 lanes cover a head (each lane 8 dims of the first half and their partners in the second
// half), so a load instruction of the wave covers the half-rows of 64 / (d/16) neighbouring heads: the token's row
// is read and written in contiguous 2*d-byte pieces.  The angles depend on the position and the dim only; every lane
// evaluates the cos / sin of its 8 dims once and reuses them for all the heads it visits.  For the usual head dims
// (LPR = d/16 a compile-time power of two) the lanes that share the same dims split the eight evaluations among
// themselves and exchange the results, so a lane evaluates one or two angles instead of eight.
template <typename T, int LPR>
__global__ void __launch_bounds__(256)
rope_kernel(const T* __restrict__ x, int64_t x_sn, int64_t x_sh, T* __restrict__ out, int64_t o_sn,
            int64_t o_sh, const int32_t* __restrict__ cu, int batch, int64_t n, int h, int d,
            const float* __restrict__ inv_freq, float attn_scale, int start, int stride, int conj) {
  typedef typename Elem<T>::vec8 vec8;
  const int lpr = LPR > 0 ? LPR : d / 16, hpw = WAVE / lpr;
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t tok = (int64_t)blockIdx.x * (256 / WAVE) + (threadIdx.x / WAVE);
  if (tok >= n) return;
  const int sub = lane % lpr, hl = lane / lpr;
  if (hl >= hpw) return;  // lanes left over where d/16 does not divide the wave
  const int s = upper_seg(cu, batch, (int)tok);
  const float pos = (float)(start + ((int)tok - cu[s]) * stride);
  // the tables are rounded to the tensor's dtype before use, as in the reference
  auto table = [&](int e, float& cv_out, float& sv_out) {
    float sv, cv;
    sincosf(pos * inv_freq[sub * 8 + e], &sv, &cv);
    cv_out = (float)(T)(cv * attn_scale);
    sv_out = (float)(T)(sv * attn_scale);
    if (conj) sv_out = -sv_out;
  };
  float c[8], sn[8];
  if constexpr (LPR > 0) {
    constexpr int HPW = WAVE / LPR;                  // lanes that hold the same dims
    constexpr int PER = HPW >= 8 ? 1 : 8 / HPW;      // evaluations per lane
    float cl[PER], sl[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) table((hl + i * HPW) % 8, cl[i], sl[i]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {  // dim e was evaluated by the lane with hl = e % HPW in its turn e / HPW
      const int src = (e % HPW) * LPR + sub;
      c[e] = __shfl(cl[HPW >= 8 ? 0 : e / HPW], src, WAVE);
      sn[e] = __shfl(sl[HPW >= 8 ? 0 : e / HPW], src, WAVE);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) table(e, c[e], sn[e]);
  }
#pragma unroll 4
  for (int head = hl; head < h; head += hpw) {
    const T* xr = x + tok * x_sn + (int64_t)head * x_sh + sub * 8;
    vec8 a = load16<vec8>(xr), b = load16<vec8>(xr + d / 2);
    vec8 oa, ob;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float x1 = (float)a[e], x2 = (float)b[e];
      oa[e] = (T)(x1 * c[e] - x2 * sn[e]);
      ob[e] = (T)(x1 * sn[e] + x2 * c[e]);
    }
    T* orow = out + tok * o_sn + (int64_t)head * o_sh + sub * 8;
    store16(orow, oa);
    store16(orow + d / 2, ob);
  }
}

// ------------------------------------------------------- linear compress ----
constexpr int LC_KC = 64;     // contraction chunk staged per step
constexpr int LC_ROWS = 128;  // compressed tokens (or tokens) per work-group

// transposing read of 8 consecutive rows r0..r0+7 of one column out of a row-major LDS tile:
// this lane supplies the address of row r0 + (lane%16)/4, columns c0 + 4*(lane%4)
template <typename T>
__device__ __forceinline__ typename Elem<T>::vec8 lds_tr8_rows(const T* p, int stride) {
  typename Elem<T>::vec4 lo = lds_read_tr4<T>(p);
  typename Elem<T>::vec4 hi = lds_read_tr4<T>(p + 4 * stride);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Forward: a work-group owns 32 compressed tokens of one head; its four waves split the window offsets k
// (wave w takes k = w, w + 4, ...), each with a private W tile in LDS and no work-group barrier inside the loop,
// and the four partial Y^T tiles are summed through LDS at the end.  (Few compressed tokens exist - a 16th of
// the sequence - so the work is spread over the offsets as well to fill the chip.)
constexpr int LCF_ROWS = 32;  // compressed tokens per work-group
constexpr int LCF_KC = 32;    // rows of W staged per step and wave

template <int D> struct LcFwdLds {
  static constexpr int WS = D + 16;                        // W tile row stride (32 B pad for the transposing reads)
  static constexpr int RS = D + 4;                         // row stride of the fp32 reduction tiles
  static constexpr int TILE_BYTES = 4 * LCF_KC * WS * 2;
  static constexpr int RED_BYTES = 4 * LCF_ROWS * RS * 4;
  static constexpr int BYTES = TILE_BYTES > RED_BYTES ? TILE_BYTES : RED_BYTES;
};

template <typename T, int D>
__global__ void __launch_bounds__(256)
lc_fwd_kernel(const T* __restrict__ x, int64_t x_sn, int64_t x_sh, const T* __restrict__ w,
              const T* __restrict__ bias, T* __restrict__ y, const int32_t* __restrict__ cu_x,
              const int32_t* __restrict__ cu_y, int nheads, int ks, int stride) {
  typedef typename Elem<T>::vec8 vec8;
  typedef typename Elem<T>::vec4 vec4;
  constexpr int WS = LcFwdLds<D>::WS, RS = LcFwdLds<D>::RS, NT = D / 32;
  constexpr int NLD = LCF_KC * (D / 8) / 64;  // 16-byte chunks of a W tile per lane
  extern __shared__ __attribute__((aligned(16))) unsigned char lc_smem[];
  const int s = blockIdx.y, h = blockIdx.z;
  const int y0 = cu_y[s], ny = cu_y[s + 1] - y0, x0 = cu_x[s];
  const int n_lo = blockIdx.x * LCF_ROWS;
  if (n_lo >= ny) return;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  T* Wt = reinterpret_cast<T*>(lc_smem) + wv * (LCF_KC * WS);
  const int n = n_lo + col;
  const bool valid = n < ny;
  const T* xrow0 = x + (int64_t)(x0 + (valid ? n : 0) * stride) * x_sn + (int64_t)h * x_sh + 8 * hh;
  const T* wh = w + (int64_t)h * ks * D * D;
  const int tr_row = (lane & 15) >> 2, tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  f32x16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
  for (int k = wv; k < ks; k += 4)
    for (int dc = 0; dc < D; dc += LCF_KC) {
      vec8 wreg[NLD];
#pragma unroll
      for (int j = 0; j < NLD; ++j) {
        const int c = lane + 64 * j, r = c / (D / 8), cc = c % (D / 8);
        wreg[j] = load16<vec8>(wh + ((int64_t)k * D + dc + r) * D + cc * 8);
      }
      vec8 xf[LCF_KC / 16];
#pragma unroll
      for (int kk = 0; kk < LCF_KC / 16; ++kk) {
        xf[kk] = zero8<T>();
        if (valid) xf[kk] = load16<vec8>(xrow0 + (int64_t)k * x_sn + dc + 16 * kk);
      }
      __builtin_amdgcn_wave_barrier();  // the previous tile has been consumed
#pragma unroll
      for (int j = 0; j < NLD; ++j) {
        const int c = lane + 64 * j, r = c / (D / 8), cc = c % (D / 8);
        store16(&Wt[r * WS + cc * 8], wreg[j]);
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int kk = 0; kk < LCF_KC / 16; ++kk)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          vec8 wf = lds_tr8_rows<T>(&Wt[(16 * kk + 8 * hh + tr_row) * WS + t * 32 + tr_col], WS);
          acc[t] = Elem<T>::mfma32(wf, xf[kk], acc[t]);
        }
    }
  // sum of the four waves' tiles: red[wave][row][dout] fp32
  __syncthreads();
  float* red = reinterpret_cast<float*>(lc_smem);
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      f32x4 v = {acc[t][4 * qd], acc[t][4 * qd + 1], acc[t][4 * qd + 2], acc[t][4 * qd + 3]};
      *reinterpret_cast<f32x4*>(&red[(wv * LCF_ROWS + col) * RS + t * 32 + 8 * qd + 4 * hh]) = v;
    }
  __syncthreads();
  for (int e = tid; e < LCF_ROWS * (D / 4); e += 256) {
    const int row = e / (D / 4), d4 = (e % (D / 4)) * 4;
    if (n_lo + row >= ny) continue;
    f32x4 sum = *reinterpret_cast<const f32x4*>(&red[row * RS + d4]);
#pragma unroll
    for (int ww = 1; ww < 4; ++ww) sum += *reinterpret_cast<const f32x4*>(&red[(ww * LCF_ROWS + row) * RS + d4]);
    vec4 out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      T r = (T)sum[i];
      if (bias) r = (T)((float)r + (float)bias[h * D + d4 + i]);
      out[i] = r;
    }
    store8(y + ((int64_t)(y0 + n_lo + row) * nheads + h) * D + d4, out);
  }
}

// bias[h, dout] = sum_{k,d} pe[h,k,d] W[h,k,d,dout]  (fp32 accumulation, rounded once).
// One work-group per (head, 8 output columns): 32 row slices x 8 columns, slices summed in a fixed order.
template <typename T>
__global__ void __launch_bounds__(256)
lc_bias_kernel(const T* __restrict__ pe, const T* __restrict__ w, T* __restrict__ bias, int kd, int d) {
  __shared__ float part[256];
  const int h = blockIdx.x, tid = threadIdx.x;
  const int c = tid & 7, slice = tid >> 3, dout = blockIdx.y * 8 + c;
  float s = 0.f;
  for (int i = slice; i < kd; i += 32) s += (float)pe[(int64_t)h * kd + i] * (float)w[((int64_t)h * kd + i) * d + dout];
  part[tid] = s;
  __syncthreads();
  if (slice == 0) {
    for (int j = 1; j < 32; ++j) s += part[j * 8 + c];
    bias[h * d + dout] = (T)s;
  }
}

// dX: one wave = 32 tokens of one phase (t % stride), so that the window offsets k_r are wave-uniform
template <typename T, int D>
__global__ void __launch_bounds__(256)
lc_dx_kernel(const T* __restrict__ dy, const T* __restrict__ w, T* __restrict__ dx,
             const int32_t* __restrict__ cu_x, const int32_t* __restrict__ cu_y, int nheads, int ks,
             int stride) {
  typedef typename Elem<T>::vec8 vec8;
  typedef typename Elem<T>::vec4 vec4;
  constexpr int NT = D / 32;
  const int s = blockIdx.y, h = blockIdx.z;
  const int x0 = cu_x[s], len = cu_x[s + 1] - x0, y0 = cu_y[s], ny = cu_y[s + 1] - y0;
  const int m_per_phase = (len + stride - 1) / stride;
  const int tiles_per_phase = (m_per_phase + LC_ROWS - 1) / LC_ROWS;
  const int phase = blockIdx.x / tiles_per_phase, mt = blockIdx.x % tiles_per_phase;
  if (phase >= stride || len == 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int m = mt * LC_ROWS + wv * 32 + col;
  const int t = phase + stride * m;
  const bool valid = t < len;
  const int nrep = ks / stride;
  f32x16 acc[NT];
#pragma unroll
  for (int i_ = 0; i_ < NT; ++i_)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i_][i] = 0.f;
  // W[h, k] ([d][dout], 2 D^2 bytes) of the step is staged in LDS: as the A operand every lane reads a different
  // row of it, which straight from global memory is 64 cache lines per load instruction
  constexpr int WS = D + 8;
  extern __shared__ __attribute__((aligned(16))) unsigned char lc_smem[];
  T* Ws = reinterpret_cast<T*>(lc_smem);
  for (int r = 0; r < nrep; ++r) {
    const int nwin = m - r, k = phase + r * stride;
    const bool ok = valid && nwin >= 0 && nwin < ny;
    const T* dyrow = dy + ((int64_t)(y0 + (ok ? nwin : 0)) * nheads + h) * D + 8 * hh;
    const T* wk = w + ((int64_t)h * ks + k) * D * D;
    vec8 yf[D / 16];
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) {
      yf[kk] = zero8<T>();
      if (ok) yf[kk] = load16<vec8>(dyrow + 16 * kk);
    }
    if (r) __syncthreads();
    for (int c = tid; c < D * (D / 8); c += 256) {
      const int row = c / (D / 8), cc = c % (D / 8);
      store16(&Ws[row * WS + cc * 8], load16<vec8>(wk + (int64_t)row * D + cc * 8));
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk)
#pragma unroll
      for (int i_ = 0; i_ < NT; ++i_) {
        vec8 wf = load16<vec8>(&Ws[(i_ * 32 + col) * WS + 16 * kk + 8 * hh]);  // A[m = d][k = dout]
        acc[i_] = Elem<T>::mfma32(wf, yf[kk], acc[i_]);
      }
  }
  if (!valid) return;
  T* xrow = dx + ((int64_t)(x0 + t) * nheads + h) * D + 4 * hh;
#pragma unroll
  for (int i_ = 0; i_ < NT; ++i_)
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      vec4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (T)acc[i_][4 * qd + e];
      store8(xrow + i_ * 32 + 8 * qd, v);
    }
}

// dbias[h, dout] = sum_n dY[n, h, dout]  (fp32)
template <typename T>
__global__ void __launch_bounds__(256)
lc_dbias_kernel(const T* __restrict__ dy, float* __restrict__ dbias, int64_t ny_total, int nheads, int d) {
  __shared__ float part[256];
  const int h = blockIdx.x, tid = threadIdx.x;
  const int c = tid & 7, slice = tid >> 3, dout = blockIdx.y * 8 + c;
  float s = 0.f;
  for (int64_t n = slice; n < ny_total; n += 32) s += (float)dy[(n * nheads + h) * d + dout];
  part[tid] = s;
  __syncthreads();
  if (slice == 0) {
    for (int j = 1; j < 32; ++j) s += part[j * 8 + c];
    dbias[h * d + dout] = s;
  }
}

// dpe[h, k, d] = sum_dout W[h,k,d,dout] dbias[h,dout]
template <typename T>
__global__ void __launch_bounds__(256)
lc_dpe_kernel(const T* __restrict__ w, const float* __restrict__ dbias, T* __restrict__ dpe, int kd, int d) {
  const int h = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= kd) return;
  const T* wr = w + ((int64_t)h * kd + i) * d;
  float s = 0.f;
  for (int o = 0; o < d; ++o) s += (float)wr[o] * dbias[h * d + o];
  dpe[(int64_t)h * kd + i] = (T)s;
}

// dW[h, k, d, dout] = sum_n x[tok(n) + k, h, d] dY[n, h, dout] (+ pe[h,k,d] dbias[h,dout])
// One work-group per (offset k, head, 128 input dims): few work-groups, each a long loop over all compressed
// tokens, so a step covers many tokens (LCW_KC) to keep enough rows in flight.  (Cutting the output dims over more
// work-groups was measured and is slower: the strided X rows, 256 bytes every kernel_stride tokens, are what the
// kernel waits for, and every cut reads them again.)
constexpr int LCW_KC = 128;
template <int D> struct LcDwLds { static constexpr int BYTES = LCW_KC * ((128 + 16) + (D + 16)) * 2; };

template <typename T, int D>
__global__ void __launch_bounds__(256)
lc_dw_kernel(const T* __restrict__ x, int64_t x_sn, int64_t x_sh, const T* __restrict__ dy,
             const T* __restrict__ pe, const float* __restrict__ dbias, T* __restrict__ dw,
             const int32_t* __restrict__ cu_x, const int32_t* __restrict__ cu_y, int batch, int nheads,
             int ks, int stride) {
  typedef typename Elem<T>::vec8 vec8;
  constexpr int LCW_DOUT = D;  // output dims per work-group
  constexpr int XS = 128 + 16, YS = LCW_DOUT + 16, NT = LCW_DOUT / 32;  // 32 B pads: conflict-free transposing reads
  constexpr int LC_KC = LCW_KC;  // compressed tokens per step of this kernel
  constexpr int YC = LCW_DOUT / 8;  // 16-byte chunks of a dY row slice
  extern __shared__ __attribute__((aligned(16))) unsigned char lcw_smem[];
  T* Xs = reinterpret_cast<T*>(lcw_smem);
  T* Ys = Xs + LC_KC * XS;
  const int k = blockIdx.x, h = blockIdx.y;
  const int dz = (blockIdx.z / (D / LCW_DOUT)) * 128, dout0 = (blockIdx.z % (D / LCW_DOUT)) * LCW_DOUT;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int ny_total = cu_y[batch];
  const int tr_row = (lane & 15) >> 2, tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  f32x16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
  // the rows of the next step travel while the current one is multiplied
  constexpr int NX = LC_KC * 16 / 256, NY = LC_KC * YC / 256;
  static_assert(LC_KC * YC % 256 == 0, "dY slice must divide over the threads");
  vec8 xr[NX], yr[NY];
  // Token of compressed row n at window offset k (-1 past the end): looked up by one thread per row of a step (a
  // search through cu_y, a chain of dependent loads) two steps ahead and handed to the 16 threads that load the
  // row through a small double-buffered LDS table, so the search is neither repeated per chunk nor part of the
  // latency of a step.
  __shared__ int tok_l[2][LC_KC];
  auto find_tokens = [&](int n0, int buf) {
    if (tid < LC_KC) {
      const int n = n0 + tid;
      int tok = -1;
      if (n < ny_total) {
        const int s = upper_seg(cu_y, batch, n);
        tok = cu_x[s] + (n - cu_y[s]) * stride + k;
      }
      tok_l[buf][tid] = tok;
    }
  };
  auto load_step = [&](int n0, int buf) {
#pragma unroll
    for (int j = 0; j < NY; ++j) {
      const int c = tid + 256 * j, r = c / YC, cc = c % YC;
      const int n = n0 + r;
      yr[j] = zero8<T>();
      if (n < ny_total) yr[j] = load16<vec8>(dy + ((int64_t)n * nheads + h) * D + dout0 + cc * 8);
    }
#pragma unroll
    for (int j = 0; j < NX; ++j) {  // X rows: 128 dims = 16 chunks
      const int c = tid + 256 * j, cc = c % 16;
      const int tok = tok_l[buf][c / 16];
      xr[j] = zero8<T>();
      if (tok >= 0) xr[j] = load16<vec8>(x + (int64_t)tok * x_sn + (int64_t)h * x_sh + dz + cc * 8);
    }
  };
  find_tokens(0, 0);
  find_tokens(LC_KC, 1);
  __syncthreads();
  load_step(0, 0);
  // step i uses table i & 1; the table of step i + 2 is written after the barriers of step i, i.e. after every
  // thread has read the same buffer for step i's rows (in the previous iteration)
  int buf = 0;
  for (int n0 = 0; n0 < ny_total; n0 += LC_KC, buf ^= 1) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NX; ++j) {
      const int c = tid + 256 * j;
      store16(&Xs[(c / 16) * XS + (c % 16) * 8], xr[j]);
    }
#pragma unroll
    for (int j = 0; j < NY; ++j) {
      const int c = tid + 256 * j;
      store16(&Ys[(c / YC) * YS + (c % YC) * 8], yr[j]);
    }
    __syncthreads();
    if (n0 + LC_KC < ny_total) {
      load_step(n0 + LC_KC, buf ^ 1);
      find_tokens(n0 + 2 * LC_KC, buf);
    }
#pragma unroll
    for (int kk = 0; kk < LC_KC / 16; ++kk) {
      vec8 xf = lds_tr8_rows<T>(&Xs[(16 * kk + 8 * hh + tr_row) * XS + wv * 32 + tr_col], XS);  // A[m = d][k = n]
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        vec8 yf = lds_tr8_rows<T>(&Ys[(16 * kk + 8 * hh + tr_row) * YS + t * 32 + tr_col], YS);  // B[k = n][dout]
        acc[t] = Elem<T>::mfma32(xf, yf, acc[t]);
      }
    }
  }
  // C layout: lane column = dout within the tile, registers = d rows
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int dd = dz + wv * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
      const int dout = dout0 + t * 32 + col;
      float v = acc[t][i];
      if (pe) v += (float)pe[((int64_t)h * ks + k) * D + dd] * dbias[h * D + dout];
      dw[(((int64_t)h * ks + k) * D + dd) * D + dout] = (T)v;
    }
}

// -------------------------------------------------------------- gate merge ----
// out[n, :] = g[n,0] a[n, :] + g[n,1] b[n, :] + g[n,2] c[n, :]  (one wave per token row, 16-byte chunks,
// fp32 sum rounded once); backward: d_a = g0 d_out (same for b, c) and d_g[n,i] = <d_out[n, :], x_i[n, :]>.
template <typename T>
__global__ void __launch_bounds__(256)
gate_merge_fwd_kernel(const T* __restrict__ a, const T* __restrict__ b, const T* __restrict__ c,
                      const T* __restrict__ gate, T* __restrict__ out, int64_t n_tokens, int row) {
  typedef typename Elem<T>::vec8 vec8;
  const int64_t n = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= n_tokens) return;
  const int lane = threadIdx.x & 63;
  const float g0 = (float)gate[n * 3], g1 = (float)gate[n * 3 + 1], g2 = (float)gate[n * 3 + 2];
  const int64_t base = n * row;
  for (int e = lane * 8; e < row; e += 512) {
    const vec8 x = load16_stream<vec8>(a + base + e), y = load16_stream<vec8>(b + base + e), z = load16_stream<vec8>(c + base + e);
    vec8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = (T)(g0 * (float)x[i] + g1 * (float)y[i] + g2 * (float)z[i]);
    store16(out + base + e, r);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
gate_merge_bwd_kernel(const T* __restrict__ d_out, const T* __restrict__ a, const T* __restrict__ b,
                      const T* __restrict__ c, const T* __restrict__ gate, T* __restrict__ d_a,
                      T* __restrict__ d_b, T* __restrict__ d_c, T* __restrict__ d_gate, int64_t n_tokens,
                      int row) {
  typedef typename Elem<T>::vec8 vec8;
  const int64_t n = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= n_tokens) return;
  const int lane = threadIdx.x & 63;
  const float g0 = (float)gate[n * 3], g1 = (float)gate[n * 3 + 1], g2 = (float)gate[n * 3 + 2];
  const int64_t base = n * row;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f;
  for (int e = lane * 8; e < row; e += 512) {
    const vec8 w = load16_stream<vec8>(d_out + base + e);
    const vec8 x = load16_stream<vec8>(a + base + e), y = load16_stream<vec8>(b + base + e), z = load16_stream<vec8>(c + base + e);
    vec8 ra, rb, rc;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float wf = (float)w[i];
      s0 += wf * (float)x[i];
      s1 += wf * (float)y[i];
      s2 += wf * (float)z[i];
      ra[i] = (T)(g0 * wf);
      rb[i] = (T)(g1 * wf);
      rc[i] = (T)(g2 * wf);
    }
    store16(d_a + base + e, ra);
    store16(d_b + base + e, rb);
    store16(d_c + base + e, rc);
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    s0 += __shfl_xor(s0, o, 64);
    s1 += __shfl_xor(s1, o, 64);
    s2 += __shfl_xor(s2, o, 64);
  }
  if (lane == 0) {
    d_gate[n * 3] = (T)s0;
    d_gate[n * 3 + 1] = (T)s1;
    d_gate[n * 3 + 2] = (T)s2;
  }
}

}  // namespace fsa

using namespace fsa;

extern "C" int fsa_rope(const void* x, void* out, int32_t dtype, int64_t x_stride_n, int64_t x_stride_h,
                        int64_t o_stride_n, int64_t o_stride_h, const int32_t* cu_seqlens, int32_t batch,
                        int64_t total_tokens, int32_t num_heads, int32_t head_dim, const float* inv_freq,
                        float attention_scaling, int32_t start, int32_t stride, int32_t inverse,
                        void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(x && out && cu_seqlens && inv_freq, "fsa_rope: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_rope: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(head_dim >= 16 && head_dim % 16 == 0 && head_dim <= 1024,
                "fsa_rope: head_dim must be a multiple of 16, at most 1024");
  FSA_CHECK_ARG(batch >= 1 && num_heads >= 1, "fsa_rope: bad sizes");
  if (total_tokens == 0) return 0;
  const unsigned grid = (unsigned)((total_tokens + 3) / 4);  // one wave per token
  ProfScope ps_("rope", stream);
#define FSA_ROPE(TT, LPR)                                                                                      \
  rope_kernel<TT, LPR><<<grid, 256, 0, stream>>>((const TT*)x, x_stride_n, x_stride_h, (TT*)out, o_stride_n,   \
                                                 o_stride_h, cu_seqlens, batch, total_tokens, num_heads,      \
                                                 head_dim, inv_freq, attention_scaling, start, stride, inverse)
#define FSA_ROPE_D(TT)                      \
  if (head_dim == 64) FSA_ROPE(TT, 4);      \
  else if (head_dim == 128) FSA_ROPE(TT, 8);  \
  else if (head_dim == 256) FSA_ROPE(TT, 16); \
  else FSA_ROPE(TT, 0)
  if (dtype == FSA_BF16) {
    FSA_ROPE_D(__bf16);
  } else {
    FSA_ROPE_D(_Float16);
  }
#undef FSA_ROPE_D
#undef FSA_ROPE
  FSA_CHECK_LAUNCH("fsa_rope");
  return 0;
}

template <typename T>
static int lc_fwd_t(const void* x, int64_t x_sn, int64_t x_sh, const void* w, const void* pe, void* bias,
                    void* y, const int32_t* cu_x, const int32_t* cu_y, int batch, int64_t max_y, int h, int d,
                    int ks, int stride, hipStream_t stream) {
  if (pe) {
    ProfScope ps_("linear_compress_bias", stream);
    lc_bias_kernel<T><<<dim3(h, d / 8), 256, 0, stream>>>((const T*)pe, (const T*)w, (T*)bias, ks * d, d);
  }
  dim3 grid((unsigned)((max_y + LCF_ROWS - 1) / LCF_ROWS), batch, h);
  const T* b = pe ? (const T*)bias : nullptr;
#define FSA_LC_FWD(DD)                                                                                          \
  {                                                                                                             \
    constexpr int lds = LcFwdLds<DD>::BYTES;                                                                    \
    if (lds > 48 * 1024) {                                                                                      \
      hipError_t e = hipFuncSetAttribute((const void*)lc_fwd_kernel<T, DD>,                                     \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);                      \
      if (e != hipSuccess) {                                                                                    \
        set_error("hipFuncSetAttribute(%d B LDS): %s", lds, hipGetErrorString(e));                              \
        return (int)e;                                                                                          \
      }                                                                                                         \
    }                                                                                                           \
    ProfScope ps_("linear_compress_fwd", stream);                                                               \
    lc_fwd_kernel<T, DD><<<grid, 256, lds, stream>>>((const T*)x, x_sn, x_sh, (const T*)w, b, (T*)y, cu_x, cu_y, \
                                                      h, ks, stride);                                           \
  }
  if (d == 64) FSA_LC_FWD(64)
  else if (d == 128) FSA_LC_FWD(128)
  else FSA_LC_FWD(256)
#undef FSA_LC_FWD
  return 0;
}

extern "C" int fsa_linear_compress_fwd(const void* x, const void* w, const void* pe, int32_t dtype,
                                       int64_t x_stride_n, int64_t x_stride_h, const int32_t* cu_seqlens_x,
                                       const int32_t* cu_seqlens_y, int32_t batch, int64_t max_seqlen_y,
                                       int32_t num_heads, int32_t head_dim, int32_t kernel_size,
                                       int32_t kernel_stride, void* y, void* bias_scratch, void* stream_) {
  FSA_CHECK_ARG(x && w && y && cu_seqlens_x && cu_seqlens_y, "fsa_linear_compress_fwd: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_linear_compress_fwd: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(head_dim == 64 || head_dim == 128 || head_dim == 256,
                "fsa_linear_compress_fwd: head_dim=%d not supported (64, 128, 256)", head_dim);
  FSA_CHECK_ARG(kernel_stride >= 1 && kernel_size % kernel_stride == 0,
                "fsa_linear_compress_fwd: kernel_size must be a multiple of kernel_stride");
  FSA_CHECK_ARG(!pe || bias_scratch, "fsa_linear_compress_fwd: bias scratch [H, D] needed with pe");
  if (max_seqlen_y <= 0) return 0;
  hipStream_t stream = (hipStream_t)stream_;
  const int rc = dtype == FSA_BF16
      ? lc_fwd_t<__bf16>(x, x_stride_n, x_stride_h, w, pe, bias_scratch, y, cu_seqlens_x, cu_seqlens_y, batch,
                         max_seqlen_y, num_heads, head_dim, kernel_size, kernel_stride, stream)
      : lc_fwd_t<_Float16>(x, x_stride_n, x_stride_h, w, pe, bias_scratch, y, cu_seqlens_x, cu_seqlens_y, batch,
                           max_seqlen_y, num_heads, head_dim, kernel_size, kernel_stride, stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_linear_compress_fwd");
  return 0;
}

template <typename T>
static int lc_bwd_t(const void* x, int64_t x_sn, int64_t x_sh, const void* w, const void* pe, const void* dy,
                    const int32_t* cu_x, const int32_t* cu_y, int batch, int64_t max_x, int64_t total_y, int h,
                    int d, int ks, int stride, void* dx, void* dw, void* dpe, float* dbias, hipStream_t stream) {
  {
    ProfScope ps_("linear_compress_dx", stream);
    const int64_t m_per_phase = (max_x + stride - 1) / stride;
    dim3 grid((unsigned)(stride * ((m_per_phase + LC_ROWS - 1) / LC_ROWS)), batch, h);
    // the grid is sized for the longest sequence; shorter sequences recompute their own tiling inside
#define FSA_LC_DX(DD)                                                                                           \
  {                                                                                                             \
    constexpr int lds = DD * (DD + 8) * 2;                                                                      \
    if (lds > 48 * 1024) {                                                                                      \
      hipError_t e = hipFuncSetAttribute((const void*)lc_dx_kernel<T, DD>,                                      \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);                      \
      if (e != hipSuccess) {                                                                                    \
        set_error("hipFuncSetAttribute(%d B LDS): %s", lds, hipGetErrorString(e));                              \
        return (int)e;                                                                                          \
      }                                                                                                         \
    }                                                                                                           \
    lc_dx_kernel<T, DD><<<grid, 256, lds, stream>>>((const T*)dy, (const T*)w, (T*)dx, cu_x, cu_y, h, ks, stride); \
  }
    if (d == 64) FSA_LC_DX(64)
    else if (d == 128) FSA_LC_DX(128)
    else FSA_LC_DX(256)
#undef FSA_LC_DX
  }
  if (pe) {
    ProfScope ps_("linear_compress_dbias", stream);
    lc_dbias_kernel<T><<<dim3(h, d / 8), 256, 0, stream>>>((const T*)dy, dbias, total_y, h, d);
    lc_dpe_kernel<T><<<dim3((ks * d + 255) / 256, h), 256, 0, stream>>>((const T*)w, dbias, (T*)dpe, ks * d, d);
  }
  {
    ProfScope ps_("linear_compress_dw", stream);
    dim3 grid(ks, h, d / 128);
    const T* pe_ = (const T*)pe;
#define FSA_LC_DW(DD)                                                                                           \
  {                                                                                                             \
    constexpr int lds = LcDwLds<DD>::BYTES;                                                                     \
    hipError_t e = hipFuncSetAttribute((const void*)lc_dw_kernel<T, DD>,                                        \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);                        \
    if (e != hipSuccess) {                                                                                      \
      set_error("hipFuncSetAttribute(%d B LDS): %s", lds, hipGetErrorString(e));                                \
      return (int)e;                                                                                            \
    }                                                                                                           \
    lc_dw_kernel<T, DD><<<grid, 256, lds, stream>>>((const T*)x, x_sn, x_sh, (const T*)dy, pe_, dbias, (T*)dw,   \
                                                     cu_x, cu_y, batch, h, ks, stride);                         \
  }
    if (d == 128) FSA_LC_DW(128)
    else FSA_LC_DW(256)
#undef FSA_LC_DW
  }
  return 0;
}

extern "C" int fsa_linear_compress_bwd(const void* x, const void* w, const void* pe, const void* dy,
                                       int32_t dtype, int64_t x_stride_n, int64_t x_stride_h,
                                       const int32_t* cu_seqlens_x, const int32_t* cu_seqlens_y,
                                       int32_t batch, int64_t max_seqlen_x, int64_t total_y,
                                       int32_t num_heads, int32_t head_dim, int32_t kernel_size,
                                       int32_t kernel_stride, void* dx, void* dw, void* dpe,
                                       float* dbias_scratch, void* stream_) {
  FSA_CHECK_ARG(x && w && dy && dx && dw && cu_seqlens_x && cu_seqlens_y, "fsa_linear_compress_bwd: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_linear_compress_bwd: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(head_dim == 128 || head_dim == 256,
                "fsa_linear_compress_bwd: head_dim=%d not supported (128, 256)", head_dim);
  FSA_CHECK_ARG(kernel_stride >= 1 && kernel_size % kernel_stride == 0,
                "fsa_linear_compress_bwd: kernel_size must be a multiple of kernel_stride");
  FSA_CHECK_ARG(!pe || (dpe && dbias_scratch), "fsa_linear_compress_bwd: dpe and dbias scratch needed with pe");
  FSA_CHECK_ARG(max_seqlen_x >= 1, "fsa_linear_compress_bwd: bad max_seqlen_x");
  hipStream_t stream = (hipStream_t)stream_;
  const int rc = dtype == FSA_BF16
      ? lc_bwd_t<__bf16>(x, x_stride_n, x_stride_h, w, pe, dy, cu_seqlens_x, cu_seqlens_y, batch, max_seqlen_x,
                         total_y, num_heads, head_dim, kernel_size, kernel_stride, dx, dw, dpe, dbias_scratch, stream)
      : lc_bwd_t<_Float16>(x, x_stride_n, x_stride_h, w, pe, dy, cu_seqlens_x, cu_seqlens_y, batch, max_seqlen_x,
                           total_y, num_heads, head_dim, kernel_size, kernel_stride, dx, dw, dpe, dbias_scratch,
                           stream);
  if (rc) return rc;
  FSA_CHECK_LAUNCH("fsa_linear_compress_bwd");
  return 0;
}

extern "C" int fsa_gate_merge_fwd(const void* a, const void* b, const void* c, const void* gate, int32_t dtype,
                                  int64_t total_tokens, int32_t row_elems, void* out, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(a && b && c && gate && out, "fsa_gate_merge_fwd: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_gate_merge_fwd: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(row_elems >= 8 && row_elems % 8 == 0, "fsa_gate_merge_fwd: row_elems must be a multiple of 8");
  if (total_tokens <= 0) return 0;
  const unsigned grid = (unsigned)((total_tokens + 3) / 4);
  ProfScope ps_("gate_merge_fwd", stream);
  if (dtype == FSA_BF16)
    gate_merge_fwd_kernel<__bf16><<<grid, 256, 0, stream>>>((const __bf16*)a, (const __bf16*)b, (const __bf16*)c,
                                                            (const __bf16*)gate, (__bf16*)out, total_tokens, row_elems);
  else
    gate_merge_fwd_kernel<_Float16><<<grid, 256, 0, stream>>>((const _Float16*)a, (const _Float16*)b,
                                                              (const _Float16*)c, (const _Float16*)gate,
                                                              (_Float16*)out, total_tokens, row_elems);
  FSA_CHECK_LAUNCH("fsa_gate_merge_fwd");
  return 0;
}

extern "C" int fsa_gate_merge_bwd(const void* d_out, const void* a, const void* b, const void* c,
                                  const void* gate, int32_t dtype, int64_t total_tokens, int32_t row_elems,
                                  void* d_a, void* d_b, void* d_c, void* d_gate, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FSA_CHECK_ARG(d_out && a && b && c && gate && d_a && d_b && d_c && d_gate, "fsa_gate_merge_bwd: null pointer");
  FSA_CHECK_ARG(dtype == FSA_BF16 || dtype == FSA_FP16, "fsa_gate_merge_bwd: dtype must be bf16 or fp16");
  FSA_CHECK_ARG(row_elems >= 8 && row_elems % 8 == 0, "fsa_gate_merge_bwd: row_elems must be a multiple of 8");
  if (total_tokens <= 0) return 0;
  const unsigned grid = (unsigned)((total_tokens + 3) / 4);
  ProfScope ps_("gate_merge_bwd", stream);
  if (dtype == FSA_BF16)
    gate_merge_bwd_kernel<__bf16><<<grid, 256, 0, stream>>>(
        (const __bf16*)d_out, (const __bf16*)a, (const __bf16*)b, (const __bf16*)c, (const __bf16*)gate,
        (__bf16*)d_a, (__bf16*)d_b, (__bf16*)d_c, (__bf16*)d_gate, total_tokens, row_elems);
  else
    gate_merge_bwd_kernel<_Float16><<<grid, 256, 0, stream>>>(
        (const _Float16*)d_out, (const _Float16*)a, (const _Float16*)b, (const _Float16*)c, (const _Float16*)gate,
        (_Float16*)d_a, (_Float16*)d_b, (_Float16*)d_c, (_Float16*)d_gate, total_tokens, row_elems);
  FSA_CHECK_LAUNCH("fsa_gate_merge_bwd");
  return 0;
}
