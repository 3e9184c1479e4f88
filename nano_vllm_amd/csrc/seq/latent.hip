// Latent attention: what a layer keeps per token is a low-rank latent c (RMS-normed) and ONE rotated key part shared by all
// heads; keys and values of a head are W_uk c and W_uv c. The attention itself runs in the latent space ("absorbed" form): the
// query of head h becomes [W_uk,h^T q_h | rotated part], the cached row [c | rotated key part] is its key and c its value, and
// W_uv,h is applied to the attention output — one shared "kv head" of size kv_rank + rot_dim for all query heads, which is the
// paged windowed attention of attn_window.hip with G = 1. This file holds what surrounds it: the norms of both latents with the
// key rotation and the cache store in one launch, and the rotation of the query parts into the assembled query rows.
//
// Rotation: `rot_dims` leading entries of the rotated part turn by pos * freq[i], i < rot_dims / 2; the pair of i is
// (2i, 2i+1), or (i, i + rot_dims / 2) with `halves`; cos and sin are both multiplied by `mag` (1 without frequency scaling).
// Angles are 32-bit products of an exact integer position and a 32-bit frequency.
#include "seq_common.h"

namespace {

template <typename T>
__device__ __forceinline__ void rotate_part(const T* __restrict__ in, T* __restrict__ out, int width, int rot_dims, int halves, float mag,
                                            const float* __restrict__ freq, float pf, int lane, int lanes) {
  const int half = rot_dims >> 1;
  for (int i = lane; i < half; i += lanes) {
    const int a = halves ? i : 2 * i, b = halves ? i + half : 2 * i + 1;
    float sn, cs;
    sincosf(pf * freq[i], &sn, &cs);
    sn *= mag;
    cs *= mag;
    const float u = ldf(in + a), v = ldf(in + b);
    stf(out + a, u * cs - v * sn);
    stf(out + b, v * cs + u * sn);
  }
  for (int c = rot_dims + lane; c < width; c += lanes) out[c] = in[c];
}

// one workgroup of two wavefronts per token: wavefront 0 norms the query latent, wavefront 1 norms the key/value latent, rotates
// the shared key part and stores both into the token's cache slot (a layer that borrows another layer's cache has no such part)
template <typename T>
__global__ __launch_bounds__(128) void latent_prep_kernel(const T* __restrict__ proj, int64_t stride, int q_col, int q_rank,
                                                          const T* __restrict__ q_norm, T* __restrict__ cq, int kv_col, int kv_rank,
                                                          int rot_dim, const T* __restrict__ kv_norm, const int64_t* __restrict__ pos,
                                                          const float* __restrict__ freq, int rot_dims, int halves, float mag, float eps,
                                                          int block_size, const int32_t* __restrict__ slots, T* __restrict__ k_cache,
                                                          T* __restrict__ v_cache) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave == 0) {
    const T* src = proj + t * stride + q_col;
    float ss = 0.f;
    for (int c = lane; c < q_rank; c += 64) {
      const float v = ldf(src + c);
      ss += v * v;
    }
    const float r = 1.f / sqrtf(wave_sum(ss) / (float)q_rank + eps);
    for (int c = lane; c < q_rank; c += 64) stf(cq + t * q_rank + c, ldf(src + c) * r * ldf(q_norm + c));
    return;
  }
  if (kv_col < 0) return;
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const T* src = proj + t * stride + kv_col;
  float ss = 0.f;
  for (int c = lane; c < kv_rank; c += 64) {
    const float v = ldf(src + c);
    ss += v * v;
  }
  const float r = 1.f / sqrtf(wave_sum(ss) / (float)kv_rank + eps);
  const int D = kv_rank + rot_dim;
  T* kc = k_cache + slot * D;
  // the latent is the leading part of the key row and, transposed inside its page ([page][kv_rank][block]), the value
  const int64_t page = slot / block_size, off = slot - page * block_size;
  T* vc = v_cache + page * kv_rank * block_size + off;
  for (int c = lane; c < kv_rank; c += 64) {
    T val;
    stf(&val, ldf(src + c) * r * ldf(kv_norm + c));
    kc[c] = val;
    vc[(int64_t)c * block_size] = val;
  }
  rotate_part(src + kv_rank, kc + kv_rank, rot_dim, rot_dims, halves, mag, freq, (float)pos[t], lane, 64);
}

// out[t, h, :width] = rotated in[t, h, :width] for every head: the rotated query parts go behind the absorbed parts
template <typename T>
__global__ void rotate_heads_kernel(const T* __restrict__ in, int64_t in_stride, int in_head, T* __restrict__ out, int64_t out_stride,
                                    int out_head, int H, int width, const int64_t* __restrict__ pos, const float* __restrict__ freq,
                                    int rot_dims, int halves, float mag) {
  const int64_t t = blockIdx.x;
  const float pf = (float)pos[t];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int h = wave; h < H; h += nw)
    rotate_part(in + t * in_stride + (int64_t)h * in_head, out + t * out_stride + (int64_t)h * out_head, width, rot_dims, halves, mag, freq,
                pf, lane, 64);
}

}  // namespace

extern "C" int nvs_latent_prep(const void* proj, int64_t stride, int dtype, int q_col, int q_rank, const void* q_norm, void* cq, int kv_col,
                               int kv_rank, int rot_dim, const void* kv_norm, const int64_t* pos, const float* rot_freq, int rot_dims,
                               int rot_halves, float rot_mag, float eps, int block_size, const int32_t* slots, void* k_cache, void* v_cache,
                               int64_t n, void* stream) {
  NVS_REQUIRE(proj && q_norm && cq && q_col >= 0 && q_rank > 0 && stride >= q_col + q_rank && n >= 0, "nvs_latent_prep: query latent %d + %d of %lld",
              q_col, q_rank, (long long)stride);
  if (kv_col >= 0) {
    NVS_REQUIRE(kv_norm && pos && slots && k_cache && v_cache && kv_rank > 0 && rot_dim >= 0 && block_size > 0 &&
                    stride >= (int64_t)kv_col + kv_rank + rot_dim,
                "nvs_latent_prep: key/value latent %d + %d + %d of %lld", kv_col, kv_rank, rot_dim, (long long)stride);
    NVS_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= rot_dim && (rot_dims == 0 || rot_freq), "nvs_latent_prep: rotation of %d of %d entries",
                rot_dims, rot_dim);
  }
  if (n == 0) return NVS_OK;
  NVS_DISPATCH(dtype, latent_prep_kernel<T><<<dim3((unsigned)n), dim3(128), 0, (hipStream_t)stream>>>(
                          (const T*)proj, stride, q_col, q_rank, (const T*)q_norm, (T*)cq, kv_col, kv_rank, rot_dim, (const T*)kv_norm, pos,
                          rot_freq, rot_dims, rot_halves, rot_mag, eps, block_size, slots, (T*)k_cache, (T*)v_cache));
  return nvs_check_launch("nvs_latent_prep");
}

extern "C" int nvs_rotate_heads(const void* in, int64_t in_stride, int in_head, void* out, int64_t out_stride, int out_head, int dtype, int H,
                                int width, const int64_t* pos, const float* rot_freq, int rot_dims, int rot_halves, float rot_mag, int64_t n,
                                void* stream) {
  NVS_REQUIRE(in && out && pos && H > 0 && width >= 0 && in_head >= width && out_head >= width && in_stride >= (int64_t)(H - 1) * in_head + width &&
                  out_stride >= (int64_t)(H - 1) * out_head + width && n >= 0,
              "nvs_rotate_heads: %d heads of %d entries", H, width);
  NVS_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= width && (rot_dims == 0 || rot_freq), "nvs_rotate_heads: rotation of %d of %d entries",
              rot_dims, width);
  if (n == 0 || width == 0) return NVS_OK;
  const int threads = H >= 4 ? 256 : 64 * H;
  NVS_DISPATCH(dtype, rotate_heads_kernel<T><<<dim3((unsigned)n), dim3(threads), 0, (hipStream_t)stream>>>(
                          (const T*)in, in_stride, in_head, (T*)out, out_stride, out_head, H, width, pos, rot_freq, rot_dims, rot_halves, rot_mag));
  return nvs_check_launch("nvs_rotate_heads");
}
