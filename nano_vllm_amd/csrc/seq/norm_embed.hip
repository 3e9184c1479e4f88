// Residual-stream kernels: embedding + sinusoid, output-side scalar RMS norms with the residual add, the final norm on
// selected rows, xIELU. The residual stream is 32-bit; a copy in the activation type feeds the next matrix product.
#include "seq_common.h"
#include <string.h>

namespace {
thread_local char g_err[512] = "";
}
void nvs_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
int nvs_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    nvs_set_error("%s: HIP launch failed: %s", what, hipGetErrorString(e));
    return NVS_ELAUNCH;
  }
  return NVS_OK;
}
extern "C" int nvs_abi_version(void) { return 5; }   // 5: norms on both sides of a sublayer, attention sinks and query temperature, the gated matrix memory, table-routed experts
extern "C" const char* nvs_last_error(void) { return g_err; }

namespace {

template <typename T>
__global__ void embed_sinusoid_kernel(const T* __restrict__ table, const int64_t* __restrict__ ids, const int64_t* __restrict__ pos,
                                      int width, float scale, float log2_base, float* __restrict__ x, T* __restrict__ xh) {
  const int64_t t = blockIdx.x;
  const int64_t id = ids[t];
  const float p = (float)pos[t];
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const int i = c >> 1;
    // base^(-2i/width) in 32-bit; the angle is the product of two 32-bit numbers
    const float inv = exp2f(-(2.f * (float)i / (float)width) * log2_base);
    const float ang = p * inv;
    const float pe = log2_base > 0.f ? ((c & 1) ? cosf(ang) : sinf(ang)) : 0.f;      // (no base: no sinusoid)
    const float v = ldf(table + id * width + c) * scale + pe;
    x[t * width + c] = v;
    if (xh) stf(xh + t * width + c, v);
  }
}

// one workgroup per token row
template <typename T>
__global__ void norm_residual_kernel(const T* __restrict__ m, const T* __restrict__ m2, const T* __restrict__ w1,
                                     const T* __restrict__ w2, const T* __restrict__ g, int width, float eps,
                                     float* __restrict__ x, T* __restrict__ xh) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float gv = ldf(g);
  float ss = 0.f;
  if (m2 == nullptr) {
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      const float v = ldf(m + t * width + c);
      ss += v * v;
    }
    const float r = rsqrtf(block_sum(ss, red) / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      const float v = x[t * width + c] + gv * (ldf(m + t * width + c) * r);
      x[t * width + c] = v;
      if (xh) stf(xh + t * width + c, v);
    }
    return;
  }
  float s2 = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float a = ldf(m + t * width + c), b = ldf(m2 + t * width + c);
    ss += a * a;
    s2 += b * b;
  }
  const float r1 = rsqrtf(block_sum(ss, red) / (float)width + eps);
  const float r2 = rsqrtf(block_sum(s2, red) / (float)width + eps);
  float s3 = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = 0.5f * (ldf(m + t * width + c) * r1 * ldf(w1 + c) + ldf(m2 + t * width + c) * r2 * ldf(w2 + c));
    s3 += v * v;
  }
  const float r3 = rsqrtf(block_sum(s3, red) / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float mm = 0.5f * (ldf(m + t * width + c) * r1 * ldf(w1 + c) + ldf(m2 + t * width + c) * r2 * ldf(w2 + c));
    const float v = x[t * width + c] + gv * (mm * r3);
    x[t * width + c] = v;
    if (xh) stf(xh + t * width + c, v);
  }
}

template <typename T>
__global__ void scalar_norm_rows_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows, int width,
                                        const T* __restrict__ g, float eps, T* __restrict__ out) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[r] : r;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = x[src * width + c];
    ss += v * v;
  }
  const float k = rsqrtf(block_sum(ss, red) / (float)width + eps) * ldf(g);
  for (int c = threadIdx.x; c < width; c += blockDim.x) stf(out + r * width + c, x[src * width + c] * k);
}

template <typename T>
__global__ void xielu_kernel(const T* __restrict__ in, const T* __restrict__ pq, float beta, int64_t numel, T* __restrict__ out) {
  const float ap = softplusf_(ldf(pq)), aq = beta + softplusf_(ldf(pq + 1));
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < numel; i += (int64_t)gridDim.x * blockDim.x) {
    const float z = ldf(in + i);
    const float v = z > 0.f ? ap * z * z + beta * z : aq * (expm1f(z) - z) + beta * z;
    stf(out + i, v);
  }
}

// Input-side ("pre") norm on the 32-bit residual: x[t] += a_mult * a[t] + b[t] first (either may be absent), then every one of
// `groups` equal parts of the row is divided by its own root mean square — or, with `center`, its mean is taken off first and
// it is divided by its standard deviation (a layer norm without bias) — and the row is multiplied by w. One workgroup per
// row; a group is served by one wavefront (several groups per wavefront, in turn, when there are more groups than wavefronts)
// or by `blockDim / 64 / groups` wavefronts together when there are fewer. With `rows` the kernel only reads:
// out[r] = norm(x[rows[r]]).
template <typename T>
__global__ void add_group_norm_kernel(float* __restrict__ x, const T* __restrict__ a, float a_mult, const float* __restrict__ b,
                                      const int32_t* __restrict__ rows, const T* __restrict__ w, int width, int groups, float eps,
                                      int center, T* __restrict__ out) {
  __shared__ float red[2][16];
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? (int64_t)rows[r] : r;
  const int gsz = width / groups, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  float* xr = x + t * width;
  const int wpg = nw > groups ? nw / groups : 1;    // wavefronts per group (the host makes nw a multiple of groups then)
  const int first = wave / wpg, step = nw / wpg, idx = (wave % wpg) * 64 + lane, stride = wpg * 64;
  for (int g = first; g < groups; g += step) {
    const int c0 = g * gsz;
    float ss = 0.f, sm = 0.f;
    for (int c = idx; c < gsz; c += stride) {
      float v = xr[c0 + c];
      if (a) v += a_mult * ldf(a + t * width + c0 + c);
      if (b) v += b[t * width + c0 + c];
      if (a || b) xr[c0 + c] = v;
      ss += v * v;
      sm += v;
    }
    if (!out) continue;                             // (uniform over the workgroup)
    float mean = 0.f;
    if (center) {                                   // the mean first, then the squared deviations (this thread wrote xr[c0 + c])
      sm = wave_sum(sm);
      if (wpg > 1) {
        if (lane == 0) red[1][wave] = sm;
        __syncthreads();
        sm = 0.f;
        for (int i = 0; i < wpg; ++i) sm += red[1][first * wpg + i];
      }
      mean = sm / (float)gsz;
      ss = 0.f;
      for (int c = idx; c < gsz; c += stride) {
        const float dv = xr[c0 + c] - mean;
        ss += dv * dv;
      }
    }
    ss = wave_sum(ss);
    if (wpg > 1) {                                  // (then every wavefront runs this loop exactly once)
      if (lane == 0) red[0][wave] = ss;
      __syncthreads();
      ss = 0.f;
      for (int i = 0; i < wpg; ++i) ss += red[0][first * wpg + i];
    }
    const float k = 1.f / sqrtf(ss / (float)gsz + eps);
    for (int c = idx; c < gsz; c += stride) stf(out + r * width + c0 + c, (xr[c0 + c] - mean) * k * ldf(w + c0 + c));
  }
}

// Norms on BOTH sides of a sublayer, on the 32-bit residual: the sublayer's output y[t] = a_mult * a[t] + a2_mult * a2[t] (a2 may be
// absent) is RMS-normed with the weight (w_off + wa) and added, x[t] += rms(y[t]) * (w_off + wa); then the NEXT sublayer's input
// out[t] = rms(x[t]) * (w_off + w). Either half may be absent (a NULL / out NULL). w_off = 1 serves weights stored as their distance
// from one. With `rows` the kernel only reads: out[r] = norm(x[rows[r]]). One workgroup per row; all sums in 32-bit.
template <typename T>
__global__ void sandwich_norm_kernel(float* __restrict__ x, const T* __restrict__ a, float a_mult, const T* __restrict__ a2, float a2_mult,
                                     const T* __restrict__ wa, const int32_t* __restrict__ rows, const T* __restrict__ w, float w_off,
                                     int width, float eps, T* __restrict__ out) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? (int64_t)rows[r] : r;
  float* xr = x + t * width;
  if (a) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      float y = a_mult * ldf(a + t * width + c);
      if (a2) y += a2_mult * ldf(a2 + t * width + c);
      ss += y * y;
    }
    const float k = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      float y = a_mult * ldf(a + t * width + c);
      if (a2) y += a2_mult * ldf(a2 + t * width + c);
      xr[c] += y * k * (w_off + ldf(wa + c));
    }
  }
  if (!out) return;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {     // (every thread reads back what it wrote itself)
    const float v = xr[c];
    ss += v * v;
  }
  const float k = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x) stf(out + r * width + c, xr[c] * k * (w_off + ldf(w + c)));
}

// logits <- cap * tanh(logits * scale / cap) (cap <= 0: logits * scale), 32-bit out
template <typename T>
__global__ void scale_softcap_kernel(const T* __restrict__ in, float scale, float cap, int64_t numel, float* __restrict__ out) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < numel; i += (int64_t)gridDim.x * blockDim.x) {
    const float z = ldf(in + i) * scale;
    out[i] = cap > 0.f ? cap * tanhf(z / cap) : z;
  }
}

int threads_for(int width) { return width >= 1024 ? 256 : (width >= 256 ? 128 : 64); }

}  // namespace

extern "C" int nvs_embed_sinusoid(const void* table, int dtype, const int64_t* ids, const int64_t* pos, int64_t n, int width,
                                  float scale, float base, float* x, void* xh, void* stream) {
  NVS_REQUIRE(table && ids && pos && x && n >= 0 && width > 0 && (base > 1.f || base == 0.f), "nvs_embed_sinusoid: bad argument");
  if (n == 0) return NVS_OK;
  NVS_DISPATCH(dtype, embed_sinusoid_kernel<T><<<dim3((unsigned)n), dim3(threads_for(width)), 0, (hipStream_t)stream>>>(
                          (const T*)table, ids, pos, width, scale, base > 1.f ? log2f(base) : 0.f, x, (T*)xh));
  return nvs_check_launch("nvs_embed_sinusoid");
}

extern "C" int nvs_norm_residual(const void* m, const void* m2, const void* w1, const void* w2, const void* g, int dtype,
                                 int64_t n, int width, float eps, float* x, void* xh, void* stream) {
  NVS_REQUIRE(m && g && x && n >= 0 && width > 0, "nvs_norm_residual: bad argument");
  NVS_REQUIRE(!m2 || (w1 && w2), "nvs_norm_residual: two branches need both channel weights");
  if (n == 0) return NVS_OK;
  NVS_DISPATCH(dtype, norm_residual_kernel<T><<<dim3((unsigned)n), dim3(threads_for(width)), 0, (hipStream_t)stream>>>(
                          (const T*)m, (const T*)m2, (const T*)w1, (const T*)w2, (const T*)g, width, eps, x, (T*)xh));
  return nvs_check_launch("nvs_norm_residual");
}

extern "C" int nvs_scalar_norm_rows(const float* x, const int32_t* rows, int64_t nrows, int width, const void* g, int dtype,
                                    float eps, void* out, void* stream) {
  NVS_REQUIRE(x && g && out && nrows >= 0 && width > 0, "nvs_scalar_norm_rows: bad argument");
  if (nrows == 0) return NVS_OK;
  NVS_DISPATCH(dtype, scalar_norm_rows_kernel<T><<<dim3((unsigned)nrows), dim3(threads_for(width)), 0, (hipStream_t)stream>>>(
                          x, rows, width, (const T*)g, eps, (T*)out));
  return nvs_check_launch("nvs_scalar_norm_rows");
}

extern "C" int nvs_xielu(const void* in, const void* pq, float beta, int dtype, int64_t numel, void* out, void* stream) {
  NVS_REQUIRE(in && pq && out && numel >= 0, "nvs_xielu: bad argument");
  if (numel == 0) return NVS_OK;
  const int64_t blocks = (numel + 255) / 256;
  NVS_DISPATCH(dtype, xielu_kernel<T><<<dim3((unsigned)(blocks > 65536 ? 65536 : blocks)), dim3(256), 0, (hipStream_t)stream>>>(
                          (const T*)in, (const T*)pq, beta, numel, (T*)out));
  return nvs_check_launch("nvs_xielu");
}

extern "C" int nvs_add_group_norm(float* x, const void* a, float a_mult, const float* b, const int32_t* rows, int64_t nrows, const void* w,
                                  int dtype, int width, int groups, float eps, int center, void* out, void* stream) {
  NVS_REQUIRE(x && nrows >= 0 && width > 0 && groups > 0 && width % groups == 0 && (!out || w), "nvs_add_group_norm: width %d groups %d",
              width, groups);
  NVS_REQUIRE(!rows || (!a && !b), "nvs_add_group_norm: selected rows are only read");
  if (nrows == 0) return NVS_OK;
  // a wavefront per group, four groups at a time; wide groups that are fewer than four are shared by 4 / groups wavefronts
  int threads = 64 * (groups < 4 ? groups : 4);
  if (groups < 4 && 4 % groups == 0 && width / groups >= 512) threads = 256;
  NVS_DISPATCH(dtype, add_group_norm_kernel<T><<<dim3((unsigned)nrows), dim3(threads), 0, (hipStream_t)stream>>>(
                          x, (const T*)a, a_mult, b, rows, (const T*)w, width, groups, eps, center, (T*)out));
  return nvs_check_launch("nvs_add_group_norm");
}

extern "C" int nvs_sandwich_norm(float* x, const void* a, float a_mult, const void* a2, float a2_mult, const void* wa, const int32_t* rows,
                                 int64_t nrows, const void* w, float w_off, int dtype, int width, float eps, void* out, void* stream) {
  NVS_REQUIRE(x && nrows >= 0 && width > 0 && (a || out) && (!a || wa) && (!a2 || a) && (!out || w), "nvs_sandwich_norm: bad argument (width %d)", width);
  NVS_REQUIRE(!rows || !a, "nvs_sandwich_norm: selected rows are only read");
  if (nrows == 0) return NVS_OK;
  NVS_DISPATCH(dtype, sandwich_norm_kernel<T><<<dim3((unsigned)nrows), dim3(threads_for(width)), 0, (hipStream_t)stream>>>(
                          x, (const T*)a, a_mult, (const T*)a2, a2_mult, (const T*)wa, rows, (const T*)w, w_off, width, eps, (T*)out));
  return nvs_check_launch("nvs_sandwich_norm");
}

extern "C" int nvs_scale_softcap(const void* in, int dtype, float scale, float cap, int64_t numel, float* out, void* stream) {
  NVS_REQUIRE(in && out && numel >= 0, "nvs_scale_softcap: bad argument");
  if (numel == 0) return NVS_OK;
  const int64_t blocks = (numel + 255) / 256;
  NVS_DISPATCH(dtype, scale_softcap_kernel<T><<<dim3((unsigned)(blocks > 65536 ? 65536 : blocks)), dim3(256), 0, (hipStream_t)stream>>>(
                          (const T*)in, scale, cap, numel, out));
  return nvs_check_launch("nvs_scale_softcap");
}
