// Version, error reporting and the head-dim padding helper of the C ABI.
#include "fsa_common.h"

#include <mutex>
#include <vector>

namespace fsa {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

struct ProfRec {
  const char* name;
  hipEvent_t start, stop;
};
static std::mutex g_prof_mu;
static bool g_prof_on = false;
static std::vector<ProfRec> g_prof;

ProfScope::ProfScope(const char* name, hipStream_t stream) : idx_(-1), stream_(stream) {
  if (!g_prof_on) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  ProfRec r;
  r.name = name;
  if (hipEventCreate(&r.start) != hipSuccess || hipEventCreate(&r.stop) != hipSuccess) return;
  (void)hipEventRecord(r.start, stream);
  g_prof.push_back(r);
  idx_ = (int)g_prof.size() - 1;
}

ProfScope::~ProfScope() {
  if (idx_ < 0) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  (void)hipEventRecord(g_prof[idx_].stop, stream_);
}

// dst[r, h, 0 .. d_dst) = src[r, h, 0 .. min(d_src, d_dst)) followed by zeros; 16-bit elements, 8 bytes per thread
__global__ void __launch_bounds__(256)
pad_head_dim_kernel(const uint16_t* __restrict__ src, int64_t src_sn, int64_t src_sh, int d_src,
                    uint16_t* __restrict__ dst, int64_t dst_sn, int64_t dst_sh, int d_dst, int64_t rows,
                    int heads) {
  const int per = d_dst / 4;
  const int64_t items = rows * heads * per;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < items; idx += (int64_t)gridDim.x * 256) {
    const int c = (int)(idx % per) * 4;
    const int64_t rh = idx / per;
    const int h = (int)(rh % heads);
    const int64_t r = rh / heads;
    const uint16_t* s = src + r * src_sn + h * src_sh + c;
    uint2 x = make_uint2(0u, 0u);
    if (c + 4 <= d_src) {
      x = *reinterpret_cast<const uint2*>(s);
    } else if (c < d_src) {  // d_src is a multiple of 4 in practice; the general tail copies element by element
      uint16_t e[4] = {0, 0, 0, 0};
      for (int i = 0; c + i < d_src; ++i) e[i] = s[i];
      x = make_uint2(e[0] | ((uint32_t)e[1] << 16), e[2] | ((uint32_t)e[3] << 16));
    }
    *reinterpret_cast<uint2*>(dst + r * dst_sn + h * dst_sh + c) = x;
  }
}
}  // namespace fsa

// 200: fsa_decode_topk gained scores_to_bf16 and fsa_decode_selattn gained seqlens (both inside their argument
// lists); 210: fsa_cmp_topk gained score_head_as_written, fsa_native_head_dim / fsa_pad_head_dim added.
extern "C" int fsa_version(void) { return 210; }

extern "C" int fsa_native_head_dim(int32_t head_dim) {
  if (head_dim < 1 || head_dim > 256) return -1;
  return head_dim <= 64 ? 64 : head_dim <= 128 ? 128 : 256;
}

extern "C" int fsa_pad_head_dim(const void* src, int64_t src_stride_n, int64_t src_stride_h, int32_t d_src,
                                void* dst, int64_t dst_stride_n, int64_t dst_stride_h, int32_t d_dst,
                                int64_t rows, int32_t heads, void* stream_) {
  FSA_CHECK_ARG(src && dst, "fsa_pad_head_dim: null pointer");
  FSA_CHECK_ARG(rows >= 1 && heads >= 1 && d_src >= 1 && d_dst >= 4 && d_dst % 4 == 0,
                "fsa_pad_head_dim: rows, heads and head dims must be positive, d_dst a multiple of 4");
  FSA_CHECK_ARG(src_stride_n >= 0 && src_stride_h >= 0 && dst_stride_n >= 0 && dst_stride_h >= 0 &&
                    (src_stride_n | src_stride_h | dst_stride_n | dst_stride_h) % 4 == 0 &&
                    ((uintptr_t)src | (uintptr_t)dst) % 8 == 0,
                "fsa_pad_head_dim: rows must be 8-byte aligned (non-negative strides, multiples of 4 elements)");
  FSA_CHECK_ARG(rows < ((int64_t)1 << 40) / heads / d_dst, "fsa_pad_head_dim: too many elements");
  const int64_t items = rows * heads * (d_dst / 4);
  const int64_t blocks = (items + 255) / 256;
  fsa::ProfScope ps_("pad_head_dim", (hipStream_t)stream_);
  fsa::pad_head_dim_kernel<<<(unsigned)(blocks < (1 << 20) ? blocks : (1 << 20)), 256, 0, (hipStream_t)stream_>>>(
      (const uint16_t*)src, src_stride_n, src_stride_h, d_src, (uint16_t*)dst, dst_stride_n, dst_stride_h, d_dst,
      rows, heads);
  FSA_CHECK_LAUNCH("fsa_pad_head_dim");
  return 0;
}
extern "C" const char* fsa_last_error(void) { return fsa::g_err; }

extern "C" int fsa_profile_enable(int on) {
  std::lock_guard<std::mutex> lk(fsa::g_prof_mu);
  for (auto& r : fsa::g_prof) {
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  fsa::g_prof.clear();
  fsa::g_prof_on = on != 0;
  return 0;
}

extern "C" int fsa_profile_count(void) {
  std::lock_guard<std::mutex> lk(fsa::g_prof_mu);
  return (int)fsa::g_prof.size();
}

extern "C" int fsa_profile_get(int i, char* name, int name_cap, float* ms) {
  std::lock_guard<std::mutex> lk(fsa::g_prof_mu);
  if (i < 0 || i >= (int)fsa::g_prof.size() || !name || name_cap <= 0 || !ms) {
    fsa::set_error("fsa_profile_get: bad index or buffer");
    return FSA_ERR_INVALID;
  }
  fsa::ProfRec& r = fsa::g_prof[i];
  hipError_t e = hipEventSynchronize(r.stop);
  if (e == hipSuccess) e = hipEventElapsedTime(ms, r.start, r.stop);
  if (e != hipSuccess) {
    fsa::set_error("fsa_profile_get: %s", hipGetErrorString(e));
    return (int)e;
  }
  snprintf(name, name_cap, "%s", r.name);
  return 0;
}
