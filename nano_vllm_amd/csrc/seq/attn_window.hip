// Paged attention with a local mask for any head size: key norm / rotation + K/V store, and the attention itself (one wavefront
// per (token row, query head): portions of prompts and single decoded tokens are the same launch). Scores, softmax and the
// output accumulation are 32-bit; the query norm, the rotation of the query and the sigmoid output gate are fused in.
// The mask is one of: a sliding window (the last `window` positions), blocks (`chunk` > 0: a query sees the keys of its own
// block of `chunk` positions, blocks counted from position 0 of the sequence), or plain causal.
#include "seq_common.h"

namespace {

constexpr int MAX_HEAD = 1024;      // scalar kernels (CH = 4 or 16 chunks of 64 entries per head); the matrix-core kernels take up to 256

// first key position the query at position p sees (both masks are monotone in p, which the tile bounds below rely on)
__device__ __forceinline__ int vis_lo(int p, int window, int chunk) {
  if (window > 0) return p - window + 1 > 0 ? p - window + 1 : 0;
  if (chunk > 0) return p - p % chunk;
  return 0;
}

// factor on the query at position p: 1 + coef * ln(floor((p + 1) / every) + 1) — a temperature that grows with the logarithm of the
// position, in steps of `every` positions (every == 0: none)
// (positions are below 2^24, so p + 1 and `every` are exact in 32-bit floats and the correctly rounded quotient has the integer
// quotient's floor: a float division instead of the long expansion of an integer one)
__device__ __forceinline__ float query_temp(int p, float coef, int every) {
  if (every <= 0) return 1.f;
  return 1.f + coef * logf(floorf((float)(p + 1) / (float)every) + 1.f);
}

// one wavefront per (token, kv head)
template <typename T, int CH>
__global__ void knorm_kvstore_kernel(const T* __restrict__ k, const T* __restrict__ v, int64_t stride, const T* __restrict__ knorm,
                                     float eps, int G, int d, int dv, int block_size, const int32_t* __restrict__ slots,
                                     const int64_t* __restrict__ pos, const float* __restrict__ rot_freq, int rot_dims,
                                     T* __restrict__ k_cache, T* __restrict__ v_cache) {
  const int64_t t = blockIdx.x;
  const int g = blockIdx.y, lane = threadIdx.x;
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const T* kp = k + t * stride + (int64_t)g * d;
  float kv[CH];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + 64 * i;
    kv[i] = c < d ? ldf(kp + c) : 0.f;
    ss += kv[i] * kv[i];
  }
  float r = 1.f;
  if (knorm) r = rsqrtf(wave_sum(ss) / (float)d + eps);
  T* kc = k_cache + (slot * G + g) * d;
  const float pf = rot_dims > 0 ? (float)pos[t] : 0.f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + 64 * i;
    float val = (knorm && c < d) ? kv[i] * r * ldf(knorm + c) : kv[i];
    // rotation of the pair (2i, 2i+1): the partner sits in the neighbouring lane
    const float other = __shfl_xor(val, 1, 64);
    if (c < rot_dims) {
      float sn, cs;
      sincosf(pf * rot_freq[c >> 1], &sn, &cs);
      val = (c & 1) ? val * cs + other * sn : val * cs - other * sn;
    }
    if (c < d) stf(kc + c, val);
  }
  const T* vp = v + t * stride + (int64_t)g * dv;
  // values are kept transposed inside a page, [page][G][dv][block]: the attention kernels read a column's consecutive tokens
  const int64_t page = slot / block_size, off = slot - page * block_size;
  T* vc = v_cache + ((page * G + g) * dv) * block_size + off;
  for (int c = lane; c < dv; c += 64) vc[(int64_t)c * block_size] = vp[c];
}

// one wavefront per (token, query head). Keys go in rounds of 64 (one per lane): score, running maximum, weights into LDS,
// then every lane accumulates its value columns over the round's keys.
template <typename T, int CH>
__global__ void window_attn_kernel(const T* __restrict__ q, int64_t q_stride, const T* __restrict__ qnorm, float eps,
                                   const T* __restrict__ gate, int64_t gate_stride, int gate_w, const T* __restrict__ k_cache,
                                   const T* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int64_t bt_stride,
                                   int block_size, const int32_t* __restrict__ cu_q, const int32_t* __restrict__ ctx0,
                                   const int32_t* __restrict__ tseq, int H, int G, int d, int dv, float scale, int window, int chunk,
                                   const float* __restrict__ rot_freq, int rot_dims, const float* __restrict__ sink, float qt_coef,
                                   int qt_every, T* __restrict__ out) {
  __shared__ float qs[CH * 64];
  __shared__ float ps[64];
  __shared__ int64_t slot_s[64];                    // element offset of (token, column 0) in the page-transposed V cache
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int s = tseq[t];
  const int64_t pos = (int64_t)ctx0[s] + (t - cu_q[s]);
  const int g = h / (H / G);
  // query (+ norm) into LDS
  {
    const T* qp = q + t * q_stride + (int64_t)h * d;
    float qv[CH];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = lane + 64 * i;
      qv[i] = c < d ? ldf(qp + c) : 0.f;
      ss += qv[i] * qv[i];
    }
    const float r = qnorm ? rsqrtf(wave_sum(ss) / (float)d + eps) : 1.f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = lane + 64 * i;
      float val = (qnorm && c < d) ? qv[i] * r * ldf(qnorm + c) : qv[i];
      const float other = __shfl_xor(val, 1, 64);   // rotation of the pair (2i, 2i+1)
      if (c < rot_dims) {
        float sn, cs;
        sincosf((float)pos * rot_freq[c >> 1], &sn, &cs);
        val = (c & 1) ? val * cs + other * sn : val * cs - other * sn;
      }
      if (c < d) qs[c] = val;
    }
  }
  __syncthreads();
  const int64_t lo = vis_lo((int)pos, window, chunk);
  const int32_t* bt = block_tables + (int64_t)s * bt_stride;
  // a sink is a score in the denominator that has no value: the running maximum and sum start from it
  float m = sink ? sink[h] : -INFINITY, l = sink ? 1.f : 0.f;
  scale *= query_temp((int)pos, qt_coef, qt_every);
  float acc[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) acc[i] = 0.f;
  for (int64_t j0 = lo; j0 <= pos; j0 += 64) {
    const int64_t j = j0 + lane;
    const bool live = j <= pos;
    float sc = -INFINITY;
    int64_t slot = 0, voff = 0;
    if (live) {
      const int64_t page = bt[j / block_size], off = j % block_size;
      slot = page * block_size + off;
      voff = ((page * G + g) * dv) * block_size + off;
      const T* kp = k_cache + (slot * G + g) * d;
      float dot = 0.f;
      for (int c = 0; c < d; ++c) dot += qs[c] * ldf(kp + c);
      sc = dot * scale;
    }
    const float mn = fmaxf(m, wave_max(sc));          // finite: lane 0 of every round is live
    const float alpha = expf(m - mn);                 // 0 in the first round without a sink (m = -inf)
    const float p = live ? expf(sc - mn) : 0.f;
    l = l * alpha + wave_sum(p);
    m = mn;
    __syncthreads();                                  // the previous round's readers are done
    ps[lane] = p;
    slot_s[lane] = voff;
    __syncthreads();
    const int cnt = (int)((pos - j0 + 1) < 64 ? (pos - j0 + 1) : 64);
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = lane + 64 * i;
      if (c < dv) {
        float a = acc[i] * alpha;
        for (int jj = 0; jj < cnt; ++jj) a += ps[jj] * ldf(v_cache + slot_s[jj] + (int64_t)c * block_size);
        acc[i] = a;
      }
    }
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + 64 * i;
    if (c < dv) {
      float o = acc[i] * inv;
      if (gate) {
        const float gv = ldf(gate + t * gate_stride + (int64_t)h * gate_w + (gate_w == 1 ? 0 : c));
        o *= 1.f / (1.f + expf(-gv));
      }
      stf(out + (t * H + h) * dv + c, o);
    }
  }
}


// ---- bf16 matrix-core form ------------------------------------------------------------------------------------------
// One wavefront per (16 consecutive queries of a portion, query head); four query tiles per workgroup, no LDS. Everything
// is computed transposed so that each lane owns ONE query (column l & 15) and the softmax statistics need two shuffles:
//   S^T[keys x queries] = K Q^T   v_mfma_f32_16x16x32_bf16, A = 16 key rows x 32 of d (16-byte loads from the K cache),
//                                 B = Q^T (normed, scaled, held in registers for the whole tile)
//   O^T[dv x queries]  += V^T P^T A = 16 value columns x 32 tokens: 16-byte loads from the page-transposed V cache,
//                                 B = P^T straight from the S^T accumulators of two key blocks
// The MFMA's contraction index may be permuted freely as long as both operands agree; the key rows of block kb are the
// tokens base + 32 (kb / 2) + 8 (i / 4) + 4 (kb % 2) + i % 4, which makes the 8 weights a lane holds after two key blocks
// the 8 CONSECUTIVE tokens its V load covers. Scores, maxima, sums and O stay 32-bit; the weights enter the second product
// as bf16, like V. d % 8 == 0, block_size % 8 == 0; d and dv are padded to the template's sizes with zero operands.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;
int g_no_lds = 0;          // tests / A-B: 1 keeps every wavefront on its own operand loads (no LDS sharing)
int g_packed_heads = 1;    // tests / A-B: 0 never packs heads into the query tiles

template <int DK, int DVB, int QT>     // d <= 32 DK, dv <= 16 DVB, QT tiles of 16 queries per wavefront (they share every K / V load)
__global__ __launch_bounds__(256) void window_attn_mfma_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ qnorm, float eps, const bf16_t* __restrict__ gate,
    int64_t gate_stride, int gate_w, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int64_t bt_stride, int block_size, const int32_t* __restrict__ cu_q,
    const int32_t* __restrict__ ctx0, int nseq, int H, int G, int d, int dv, float scale, int window, int chunk,
    const float* __restrict__ rot_freq, int rot_dims, const float* __restrict__ sink, float qt_coef, int qt_every,
    int bs_shift, bf16_t* __restrict__ out) {
  constexpr int QW = 16 * QT;                       // queries per wavefront
  const int lane = threadIdx.x & 63, qi = lane & 15, gq = lane >> 4;
  int tile = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int h = blockIdx.y, g = h / (H / G);
  int s = 0, len = 0;
  for (; s < nseq; ++s) {
    len = cu_q[s + 1] - cu_q[s];
    const int tiles = (len + QW - 1) / QW;
    if (tile < tiles) break;
    tile -= tiles;
  }
  if (s >= nseq) return;                            // (no workgroup barrier below: a wavefront may leave alone)
  // positions fit 32 bits (the engine's tables do); page and offset of a token by shift and mask when pages are a power of two
  const int c0 = ctx0[s];
  const int p_first = c0 + tile * QW;
  const int p_last = c0 + (tile * QW + QW - 1 < len ? tile * QW + QW - 1 : len - 1);
  const int bs_mask = block_size - 1;

  // Q^T operands: lane holds d elements [32 c + 8 gq, + 8) of query qi of each tile, normed and scaled
  bf16x8_t qb[QT][DK];
  bool valid_q[QT];
  int64_t row[QT];
  int pos[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int rel = tile * QW + t * 16 + qi;
    valid_q[t] = rel < len;
    row[t] = (int64_t)cu_q[s] + (valid_q[t] ? rel : len - 1);
    pos[t] = c0 + rel;
    float qv[DK][8];
    float ss = 0.f;
    const bf16_t* qp = q + row[t] * q_stride + (int64_t)h * d;
#pragma unroll
    for (int c = 0; c < DK; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int col = c * 32 + gq * 8 + e;
        qv[c][e] = col < d ? (float)qp[col] : 0.f;
        ss += qv[c][e] * qv[c][e];
      }
    float r = scale * query_temp(pos[t], qt_coef, qt_every);
    if (qnorm) {
      ss += __shfl_xor(ss, 16, 64);
      ss += __shfl_xor(ss, 32, 64);
      r *= rsqrtf(ss / (float)d + eps);
    }
#pragma unroll
    for (int c = 0; c < DK; ++c)
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const int col = c * 32 + gq * 8 + e;
        const float w0 = (qnorm && col < d) ? (float)qnorm[col] : 1.f;
        const float w1 = (qnorm && col + 1 < d) ? (float)qnorm[col + 1] : 1.f;
        float a = qv[c][e] * r * w0, b = qv[c][e + 1] * r * w1;
        if (col < rot_dims) {                        // the pair (2i, 2i+1) turns by pos * freq[i]; both halves are this lane's
          float sn, cs;
          sincosf((float)pos[t] * rot_freq[col >> 1], &sn, &cs);
          const float a2 = a * cs - b * sn;
          b = b * cs + a * sn;
          a = a2;
        }
        qb[t][c][e] = (bf16_t)a;
        qb[t][c][e + 1] = (bf16_t)b;
      }
  }
  const int lo = vis_lo(p_first, window, chunk);
  const int lo_hi = vis_lo(c0 + tile * QW + QW - 1, window, chunk);      // the tile's last query sees the least far back
  const int32_t* bt = block_tables + (int64_t)s * bt_stride;
  const float sink_m = sink ? sink[h] : -1e30f, sink_l = sink && gq == 0 ? 1.f : 0.f;      // (see the LDS form below)
  float m[QT], lsum[QT];
  f32x4_t oacc[QT][DVB];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m[t] = sink_m;
    lsum[t] = sink_l;
#pragma unroll
    for (int db = 0; db < DVB; ++db) oacc[t][db] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  const bf16x8_t zero8 = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});

  for (int j0 = lo & ~31; j0 <= p_last; j0 += 64) {
    // every query of the wavefront sees all 64 tokens of the round: no masks (most rounds of a long window)
    const bool interior = j0 + 63 <= p_first && j0 >= lo_hi;
    // ---- S^T for 64 tokens: 4 key blocks, every K fragment feeds all QT tiles
    f32x4_t sacc[QT][4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
      for (int t = 0; t < QT; ++t) sacc[t][kb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const int j = j0 + (kb >> 1) * 32 + (qi >> 2) * 8 + (kb & 1) * 4 + (qi & 3);          // the token of this lane's A row
      const bool have = j <= p_last;
      const bf16_t* kp = k_cache;
      if (have) {
        const int pg = bs_shift >= 0 ? j >> bs_shift : j / block_size;
        const int off = bs_shift >= 0 ? j & bs_mask : j - pg * block_size;
        kp += (((int64_t)bt[pg] * block_size + off) * G + g) * d + gq * 8;
      }
#pragma unroll
      for (int c = 0; c < DK; ++c) {
        bf16x8_t a = zero8;
        if (have && c * 32 + gq * 8 < d) a = *(const bf16x8_t*)(kp + c * 32);
#pragma unroll
        for (int t = 0; t < QT; ++t) sacc[t][kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qb[t][c], sacc[t][kb], 0, 0, 0);
      }
    }
    // ---- mask, running maximum, weights (this lane: query qi of tile t, tokens 32 (kb/2) + 8 gq + 4 (kb%2) + r)
    bf16x8_t pb[QT][2];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float mx = m[t];
      unsigned okbits = 0xffffu;                     // bit 4 kb + r: the token is visible to this lane's query
      if (!interior) {
        okbits = 0u;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int j = j0 + (kb >> 1) * 32 + gq * 8 + (kb & 1) * 4 + r;
            const bool ok = valid_q[t] && j <= pos[t] && j >= vis_lo(pos[t], window, chunk);
            okbits |= ok ? (1u << (kb * 4 + r)) : 0u;
          }
      }
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (okbits & (1u << (kb * 4 + r))) mx = fmaxf(mx, sacc[t][kb][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float alpha = __expf(m[t] - mx);
      m[t] = mx;
      float ls = lsum[t] * alpha;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float p = (okbits & (1u << (kb * 4 + r))) ? __expf(sacc[t][kb][r] - mx) : 0.f;
          ls += p;
          pb[t][kb >> 1][(kb & 1) * 4 + r] = (bf16_t)p;
        }
      lsum[t] = ls;
      if (__ballot(alpha != 1.f) != 0ull) {          // the maximum moved for some query of the tile
#pragma unroll
        for (int db = 0; db < DVB; ++db) oacc[t][db] *= alpha;
      }
    }
    // ---- O^T += V^T P^T: two groups of 32 tokens, every V fragment feeds all QT tiles
#pragma unroll
    for (int mg = 0; mg < 2; ++mg) {
      const int jb = j0 + mg * 32 + gq * 8;                                                 // 8 consecutive tokens, one page
      const bool have = jb <= p_last;
      const bf16_t* vp = v_cache;
      if (have) {
        const int pg = bs_shift >= 0 ? jb >> bs_shift : jb / block_size;
        const int off = bs_shift >= 0 ? jb & bs_mask : jb - pg * block_size;
        vp += (((int64_t)bt[pg] * G + g) * dv) * block_size + off;
      }
#pragma unroll
      for (int db = 0; db < DVB; ++db) {
        const int col = db * 16 + qi;
        bf16x8_t a = zero8;
        if (have && col < dv) a = *(const bf16x8_t*)(vp + (int64_t)col * block_size);
#pragma unroll
        for (int t = 0; t < QT; ++t) oacc[t][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[t][mg], oacc[t][db], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    float ls = lsum[t];
    ls += __shfl_xor(ls, 16, 64);
    ls += __shfl_xor(ls, 32, 64);
    if (!valid_q[t]) continue;
    const float inv = 1.f / ls;
    bf16_t* op = out + ((int64_t)row[t] * H + h) * dv;
    const bf16_t* gp = gate ? gate + row[t] * gate_stride + (int64_t)h * gate_w : nullptr;
#pragma unroll
    for (int db = 0; db < DVB; ++db)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int c = db * 16 + gq * 4 + r;
        if (c < dv) {
          float o = oacc[t][db][r] * inv;
          if (gp) o *= 1.f / (1.f + expf(-(float)gp[gate_w == 1 ? 0 : c]));
          op[c] = (bf16_t)o;
        }
      }
  }
}

// ---- the same, with the K / V tiles of a round shared through LDS ------------------------------------------------------
// A workgroup of four wavefronts serves ONE kv head: `hw` query heads of its group times 4 / hw query tiles, so every K / V
// byte is fetched from the caches once per workgroup and round instead of once per wavefront (4x less traffic; with grouped
// query heads the sharing is across heads, which also holds when every portion is a single decoded token). All threads load
// the round's 64 tokens with coalesced 16-byte loads — the NEXT round's loads are issued before the current round is
// computed — K as [token][d], V as [column][token]; the MFMA operands are 16-byte LDS reads. Softmax, masks and the token
// permutation are those of the kernel above.
template <int DK, int DVB, int QT>
__global__ __launch_bounds__(256) void window_attn_mfma_lds_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ qnorm, float eps, const bf16_t* __restrict__ gate,
    int64_t gate_stride, int gate_w, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int64_t bt_stride, int block_size, const int32_t* __restrict__ cu_q,
    const int32_t* __restrict__ ctx0, int nseq, int H, int G, int d, int dv, float scale, int window, int chunk,
    const float* __restrict__ rot_freq, int rot_dims, const float* __restrict__ sink, float qt_coef, int qt_every,
    int bs_shift, int hw, bf16_t* __restrict__ out) {
  constexpr int QW = 16 * QT, KP = 32 * DK + 8, VP = 64 + 8, VU = DVB / 2;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[64][KP];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[16 * DVB][VP];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, qi = lane & 15, gq = lane >> 4;
  // hw == 0 ("packed", QT == 1): the workgroup serves ONE token and the rows of a wavefront's query tile are 16 HEADS of the kv
  // group at that token (64 heads per workgroup) — for steps of single tokens with many query heads per kv head, where a
  // tile of 16 consecutive positions would hold one query.
  const bool packed = hw == 0;
  const int hpg = H / G, chunks = packed ? (hpg + 63) / 64 : hpg / hw;
  const int g = blockIdx.y / chunks;
  const int hl0 = packed ? (blockIdx.y % chunks) * 64 + wave * 16 : (blockIdx.y % chunks) * hw + (wave % hw);   // the wavefront's first head in the group
  const int BQ = packed ? 1 : (4 / hw) * QW;       // queries (positions) of the workgroup
  int btile = blockIdx.x, s = 0, len = 0;
  for (; s < nseq; ++s) {
    len = cu_q[s + 1] - cu_q[s];
    const int tiles = (len + BQ - 1) / BQ;
    if (btile < tiles) break;
    btile -= tiles;
  }
  if (s >= nseq) return;                            // the whole workgroup leaves
  const int c0 = ctx0[s];
  const int rel0 = packed ? btile : btile * BQ + (wave / hw) * QW;   // this wavefront's first query inside the portion (may lie beyond its end)
  const int p_first = c0 + rel0, p_hi = packed ? p_first : c0 + rel0 + QW - 1;
  const bool idle = packed ? hl0 >= hpg : rel0 >= len;               // a wavefront without queries only helps to load
  const int b_first = c0 + btile * BQ;
  const int b_last = c0 + (btile * BQ + BQ - 1 < len ? btile * BQ + BQ - 1 : len - 1);
  const int bs_mask = block_size - 1;
  const int32_t* bt = block_tables + (int64_t)s * bt_stride;

  bf16x8_t qb[QT][DK];
  bool valid_q[QT];
  int64_t row[QT];
  int pos[QT], hq[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int rel = packed ? rel0 : rel0 + t * 16 + qi;
    const int hl = packed ? hl0 + qi : hl0;
    valid_q[t] = rel < len && hl < hpg;
    hq[t] = g * hpg + (hl < hpg ? hl : hpg - 1);
    row[t] = (int64_t)cu_q[s] + (rel < len ? rel : len - 1);
    pos[t] = c0 + rel;
    float qv[DK][8];
    float ss = 0.f;
    const bf16_t* qp = q + row[t] * q_stride + (int64_t)hq[t] * d;
#pragma unroll
    for (int c = 0; c < DK; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int col = c * 32 + gq * 8 + e;
        qv[c][e] = col < d ? (float)qp[col] : 0.f;
        ss += qv[c][e] * qv[c][e];
      }
    float r = scale * query_temp(pos[t], qt_coef, qt_every);
    if (qnorm) {
      ss += __shfl_xor(ss, 16, 64);
      ss += __shfl_xor(ss, 32, 64);
      r *= rsqrtf(ss / (float)d + eps);
    }
#pragma unroll
    for (int c = 0; c < DK; ++c)
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const int col = c * 32 + gq * 8 + e;
        const float w0 = (qnorm && col < d) ? (float)qnorm[col] : 1.f;
        const float w1 = (qnorm && col + 1 < d) ? (float)qnorm[col + 1] : 1.f;
        float a = qv[c][e] * r * w0, b = qv[c][e + 1] * r * w1;
        if (col < rot_dims) {                        // the pair (2i, 2i+1) turns by pos * freq[i]; both halves are this lane's
          float sn, cs;
          sincosf((float)pos[t] * rot_freq[col >> 1], &sn, &cs);
          const float a2 = a * cs - b * sn;
          b = b * cs + a * sn;
          a = a2;
        }
        qb[t][c][e] = (bf16_t)a;
        qb[t][c][e + 1] = (bf16_t)b;
      }
  }
  // a sink: a score in the denominator without a value; the running maximum and sum start from it (the sum once per query: in
  // the lanes with gq 0). All tiles of a wavefront belong to one head, except in the packed form, which has one tile.
  const float sink_m = sink ? sink[hq[0]] : -1e30f, sink_l = sink && gq == 0 ? 1.f : 0.f;
  float m[QT], lsum[QT];
  f32x4_t oacc[QT][DVB];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m[t] = sink_m;
    lsum[t] = sink_l;
#pragma unroll
    for (int db = 0; db < DVB; ++db) oacc[t][db] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  const u32x4_t zero4 = u32x4_t{0u, 0u, 0u, 0u};
  // staging: thread -> DK 16-byte units of K (token, 8 of d) and VU units of V (column, 8 tokens)
  u32x4_t kf[DK], vf[VU];
  // page ids are looked up one round ahead of the loads that use them: a round's loads then depend on nothing in flight
  int pgk[DK], pgv;
  auto lookup = [&](int j0) {
#pragma unroll
    for (int i = 0; i < DK; ++i) {
      const int j = j0 + (tid + i * 256) / (4 * DK);
      pgk[i] = j <= b_last ? bt[bs_shift >= 0 ? j >> bs_shift : j / block_size] : 0;
    }
    const int j = j0 + (tid & 7) * 8;
    pgv = j <= b_last ? bt[bs_shift >= 0 ? j >> bs_shift : j / block_size] : 0;
  };
  auto fetch = [&](int j0) {
#pragma unroll
    for (int i = 0; i < DK; ++i) {
      const int u = tid + i * 256, tok = u / (4 * DK), part = u - tok * (4 * DK);
      const int j = j0 + tok;
      kf[i] = zero4;
      if (j <= b_last && part * 8 < d) {
        const int off = bs_shift >= 0 ? j & bs_mask : j % block_size;
        kf[i] = *(const u32x4_t*)(k_cache + (((int64_t)pgk[i] * block_size + off) * G + g) * d + part * 8);
      }
    }
#pragma unroll
    for (int i = 0; i < VU; ++i) {
      const int u = tid + i * 256, col = u >> 3, grp = u & 7;
      const int j = j0 + grp * 8;
      vf[i] = zero4;
      if (j <= b_last && col < dv) {
        const int off = bs_shift >= 0 ? j & bs_mask : j % block_size;
        vf[i] = *(const u32x4_t*)(v_cache + (((int64_t)pgv * G + g) * dv + col) * block_size + off);
      }
    }
  };
  const int lo = vis_lo(b_first, window, chunk);
  const int lo_first = vis_lo(p_first, window, chunk), lo_hi = vis_lo(p_hi, window, chunk);
  int j0 = lo & ~31;
  lookup(j0);
  fetch(j0);
  lookup(j0 + 64);
  for (; j0 <= b_last; j0 += 64) {
    __syncthreads();                                // the previous round's readers are done
#pragma unroll
    for (int i = 0; i < DK; ++i) {
      const int u = tid + i * 256, tok = u / (4 * DK), part = u - tok * (4 * DK);
      *(u32x4_t*)&Ks[tok][part * 8] = kf[i];
    }
#pragma unroll
    for (int i = 0; i < VU; ++i) {
      const int u = tid + i * 256, col = u >> 3, grp = u & 7;
      *(u32x4_t*)&Vs[col][grp * 8] = vf[i];
    }
    __syncthreads();
    if (j0 + 64 <= b_last) {
      fetch(j0 + 64);
      lookup(j0 + 128);
    }
    // a wavefront whose queries all lie before the round's tokens (or beyond the portion) has nothing to add
    if (j0 > p_hi || idle || j0 + 63 < lo_first) continue;
    const bool interior = j0 + 63 <= p_first && j0 >= lo_hi;
    f32x4_t sacc[QT][4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
      for (int t = 0; t < QT; ++t) sacc[t][kb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const int tok = (kb >> 1) * 32 + (qi >> 2) * 8 + (kb & 1) * 4 + (qi & 3);
#pragma unroll
      for (int c = 0; c < DK; ++c) {
        const bf16x8_t a = *(const bf16x8_t*)&Ks[tok][c * 32 + gq * 8];
#pragma unroll
        for (int t = 0; t < QT; ++t) sacc[t][kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qb[t][c], sacc[t][kb], 0, 0, 0);
      }
    }
    bf16x8_t pb[QT][2];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float mx = m[t];
      unsigned okbits = 0xffffu;
      if (!interior) {
        okbits = 0u;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int j = j0 + (kb >> 1) * 32 + gq * 8 + (kb & 1) * 4 + r;
            const bool ok = valid_q[t] && j <= pos[t] && j >= vis_lo(pos[t], window, chunk);
            okbits |= ok ? (1u << (kb * 4 + r)) : 0u;
          }
      }
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (okbits & (1u << (kb * 4 + r))) mx = fmaxf(mx, sacc[t][kb][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float alpha = __expf(m[t] - mx);
      m[t] = mx;
      float ls = lsum[t] * alpha;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float p = (okbits & (1u << (kb * 4 + r))) ? __expf(sacc[t][kb][r] - mx) : 0.f;
          ls += p;
          pb[t][kb >> 1][(kb & 1) * 4 + r] = (bf16_t)p;
        }
      lsum[t] = ls;
      if (__ballot(alpha != 1.f) != 0ull) {
#pragma unroll
        for (int db = 0; db < DVB; ++db) oacc[t][db] *= alpha;
      }
    }
#pragma unroll
    for (int mg = 0; mg < 2; ++mg)
#pragma unroll
      for (int db = 0; db < DVB; ++db) {
        const bf16x8_t a = *(const bf16x8_t*)&Vs[db * 16 + qi][mg * 32 + gq * 8];
#pragma unroll
        for (int t = 0; t < QT; ++t) oacc[t][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[t][mg], oacc[t][db], 0, 0, 0);
      }
  }
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    float ls = lsum[t];
    ls += __shfl_xor(ls, 16, 64);
    ls += __shfl_xor(ls, 32, 64);
    if (!valid_q[t]) continue;
    const float inv = 1.f / ls;
    bf16_t* op = out + ((int64_t)row[t] * H + hq[t]) * dv;
    const bf16_t* gp = gate ? gate + row[t] * gate_stride + (int64_t)hq[t] * gate_w : nullptr;
#pragma unroll
    for (int db = 0; db < DVB; ++db)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int c = db * 16 + gq * 4 + r;
        if (c < dv) {
          float o = oacc[t][db][r] * inv;
          if (gp) o *= 1.f / (1.f + expf(-(float)gp[gate_w == 1 ? 0 : c]));
          op[c] = (bf16_t)o;
        }
      }
  }
}

template <int DK, int DVB, int QT>
void launch_mfma_qt(const void* q, int64_t q_stride, const void* qnorm, float eps, const void* gate, int64_t gate_stride, int gate_w,
                    const void* k_cache, const void* v_cache, const int32_t* block_tables, int64_t bt_stride, int block_size,
                    const int32_t* cu_q, const int32_t* ctx0, int nseq, int64_t n, int H, int G, int d, int dv, float scale, int window,
                    int chunk, const float* rot_freq, int rot_dims, const float* sink, float qt_coef, int qt_every, void* out, hipStream_t stream) {
  int bs_shift = -1;
  for (int b = 0; b < 31; ++b)
    if ((1 << b) == block_size) bs_shift = b;
  if constexpr (64 * (32 * DK + 8) * 2 + 16 * DVB * 72 * 2 <= 160 * 1024) {      // (every size does: gfx950 has 160 KB of LDS per CU)
    if (!g_no_lds) {
      const int hpg = H / G;
      if constexpr (QT == 1) {
        // steps of (mostly) single tokens with many query heads per kv head: heads, not positions, fill the query tiles
        if (hpg >= 8 && 4 * n <= (int64_t)nseq * hpg && g_packed_heads) {
          window_attn_mfma_lds_kernel<DK, DVB, 1><<<dim3((unsigned)n, (unsigned)(G * ((hpg + 63) / 64))), dim3(256), 0, stream>>>(
              (const bf16_t*)q, q_stride, (const bf16_t*)qnorm, eps, (const bf16_t*)gate, gate_stride, gate_w, (const bf16_t*)k_cache,
              (const bf16_t*)v_cache, block_tables, bt_stride, block_size, cu_q, ctx0, nseq, H, G, d, dv, scale, window, chunk, rot_freq,
              rot_dims, sink, qt_coef, qt_every, bs_shift, 0, (bf16_t*)out);
          return;
        }
      }
      const int hw = hpg % 4 == 0 ? 4 : (hpg % 2 == 0 ? 2 : 1);
      const int bq = (4 / hw) * 16 * QT;
      const int64_t btiles = n / bq + nseq;         // an upper bound: every portion may end with a partial tile
      window_attn_mfma_lds_kernel<DK, DVB, QT><<<dim3((unsigned)btiles, (unsigned)(G * (hpg / hw))), dim3(256), 0, stream>>>(
          (const bf16_t*)q, q_stride, (const bf16_t*)qnorm, eps, (const bf16_t*)gate, gate_stride, gate_w, (const bf16_t*)k_cache,
          (const bf16_t*)v_cache, block_tables, bt_stride, block_size, cu_q, ctx0, nseq, H, G, d, dv, scale, window, chunk, rot_freq,
          rot_dims, sink, qt_coef, qt_every, bs_shift, hw, (bf16_t*)out);
      return;
    }
  }
  const int64_t tiles = n / (16 * QT) + nseq;       // an upper bound: every portion may end with a partial tile
  window_attn_mfma_kernel<DK, DVB, QT><<<dim3((unsigned)((tiles + 3) / 4), H), dim3(256), 0, stream>>>(
      (const bf16_t*)q, q_stride, (const bf16_t*)qnorm, eps, (const bf16_t*)gate, gate_stride, gate_w, (const bf16_t*)k_cache,
      (const bf16_t*)v_cache, block_tables, bt_stride, block_size, cu_q, ctx0, nseq, H, G, d, dv, scale, window, chunk, rot_freq, rot_dims,
      sink, qt_coef, qt_every, bs_shift, (bf16_t*)out);
}

// Long portions (prefill) put two tiles of 16 queries on a wavefront: half the K / V bytes through the vector cache per
// MFMA; steps of short portions (decoding) keep one tile, which gives more wavefronts.
template <int DK, int DVB>
void launch_mfma(const void* q, int64_t q_stride, const void* qnorm, float eps, const void* gate, int64_t gate_stride, int gate_w,
                 const void* k_cache, const void* v_cache, const int32_t* block_tables, int64_t bt_stride, int block_size,
                 const int32_t* cu_q, const int32_t* ctx0, int nseq, int64_t n, int H, int G, int d, int dv, float scale, int window,
                 int chunk, const float* rot_freq, int rot_dims, const float* sink, float qt_coef, int qt_every, void* out, hipStream_t stream) {
  if (n >= 32ll * nseq)
    launch_mfma_qt<DK, DVB, 2>(q, q_stride, qnorm, eps, gate, gate_stride, gate_w, k_cache, v_cache, block_tables, bt_stride, block_size, cu_q,
                               ctx0, nseq, n, H, G, d, dv, scale, window, chunk, rot_freq, rot_dims, sink, qt_coef, qt_every, out, stream);
  else
    launch_mfma_qt<DK, DVB, 1>(q, q_stride, qnorm, eps, gate, gate_stride, gate_w, k_cache, v_cache, block_tables, bt_stride, block_size, cu_q,
                               ctx0, nseq, n, H, G, d, dv, scale, window, chunk, rot_freq, rot_dims, sink, qt_coef, qt_every, out, stream);
}
}  // namespace

static int g_force_scalar = 0;
/* tests: 1 routes bf16 calls through the scalar kernel as well */
extern "C" void nvs_window_attn_force_scalar(int on) {
  g_force_scalar = on == 1;
  g_no_lds = on == 2;
  g_packed_heads = on != 3;
}

extern "C" int nvs_knorm_kvstore(const void* k, const void* v, int64_t stride, int dtype, const void* knorm, float eps, int G, int d,
                                 int dv, int block_size, const int32_t* slots, const int64_t* pos, const float* rot_freq, int rot_dims,
                                 int64_t n, void* k_cache, void* v_cache, void* stream) {
  NVS_REQUIRE(k && v && slots && k_cache && v_cache, "nvs_knorm_kvstore: null argument");
  NVS_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= d && (rot_dims == 0 || (pos && rot_freq)),
              "nvs_knorm_kvstore: rotation of %d of %d dimensions", rot_dims, d);
  NVS_REQUIRE(G > 0 && G <= 65535 && d > 0 && d <= MAX_HEAD && dv > 0 && dv <= MAX_HEAD && n >= 0 && block_size > 0,
              "nvs_knorm_kvstore: G %d d %d dv %d", G, d, dv);
  if (n == 0) return NVS_OK;
  if (d <= 256 && dv <= 256)
    NVS_DISPATCH(dtype, knorm_kvstore_kernel<T, 4><<<dim3((unsigned)n, G), dim3(64), 0, (hipStream_t)stream>>>(
                            (const T*)k, (const T*)v, stride, (const T*)knorm, eps, G, d, dv, block_size, slots, pos, rot_freq, rot_dims,
                            (T*)k_cache, (T*)v_cache));
  else
    NVS_DISPATCH(dtype, knorm_kvstore_kernel<T, 16><<<dim3((unsigned)n, G), dim3(64), 0, (hipStream_t)stream>>>(
                            (const T*)k, (const T*)v, stride, (const T*)knorm, eps, G, d, dv, block_size, slots, pos, rot_freq, rot_dims,
                            (T*)k_cache, (T*)v_cache));
  return nvs_check_launch("nvs_knorm_kvstore");
}

extern "C" int nvs_window_attn(const void* q, int64_t q_stride, const void* qnorm, float eps, const void* gate, int64_t gate_stride,
                               int gate_per_head, int dtype, const void* k_cache, const void* v_cache, const int32_t* block_tables, int64_t bt_stride,
                               int block_size, const int32_t* cu_q, const int32_t* ctx0, const int32_t* tseq, int nseq, int64_t n, int H,
                               int G, int d, int dv, float scale, int window, int chunk, const float* rot_freq, int rot_dims, const float* sink,
                               float qt_coef, int qt_every, void* out, void* stream) {
  NVS_REQUIRE(qt_every >= 0, "nvs_window_attn: a query temperature every %d positions", qt_every);
  NVS_REQUIRE(q && k_cache && v_cache && block_tables && cu_q && ctx0 && tseq && out, "nvs_window_attn: null argument");
  NVS_REQUIRE(!(window > 0 && chunk > 0), "nvs_window_attn: a window (%d) and blocks (%d) together", window, chunk);
  NVS_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= d && (rot_dims == 0 || rot_freq),
              "nvs_window_attn: rotation of %d of %d dimensions", rot_dims, d);
  NVS_REQUIRE(H > 0 && H <= 65535 && G > 0 && H % G == 0 && d > 0 && d <= MAX_HEAD && dv > 0 && dv <= MAX_HEAD && block_size > 0 && n >= 0,
              "nvs_window_attn: H %d G %d d %d dv %d block %d", H, G, d, dv, block_size);
  if (n == 0 || nseq == 0) return NVS_OK;
  const int gate_w = gate_per_head ? 1 : dv;         // gate entries per head: one for the whole head, or one per value column
  if (dtype == NVS_BF16 && d % 8 == 0 && d <= 256 && dv <= 256 && block_size % 8 == 0 && !g_force_scalar) {
    const int dk = d <= 64 ? 2 : (d <= 128 ? 4 : 8), dvb = dv <= 64 ? 4 : (dv <= 128 ? 8 : (dv <= 192 && d > 128 ? 12 : 16));
#define NVS_MFMA_CASE(DK, DVB)                                                                                                  \
  if (dk == DK && dvb == DVB)                                                                                                   \
    launch_mfma<DK, DVB>(q, q_stride, qnorm, eps, gate, gate_stride, gate_w, k_cache, v_cache, block_tables, bt_stride, block_size, cu_q, \
                         ctx0, nseq, n, H, G, d, dv, scale, window, chunk, rot_freq, rot_dims, sink, qt_coef, qt_every, out, (hipStream_t)stream);
    NVS_MFMA_CASE(2, 4) NVS_MFMA_CASE(2, 8) NVS_MFMA_CASE(2, 16) NVS_MFMA_CASE(4, 4) NVS_MFMA_CASE(4, 8) NVS_MFMA_CASE(4, 16)
    NVS_MFMA_CASE(8, 4) NVS_MFMA_CASE(8, 8) NVS_MFMA_CASE(8, 12) NVS_MFMA_CASE(8, 16)
#undef NVS_MFMA_CASE
    return nvs_check_launch("nvs_window_attn (matrix cores)");
  }
  if (d <= 256 && dv <= 256)
    NVS_DISPATCH(dtype, window_attn_kernel<T, 4><<<dim3((unsigned)n, H), dim3(64), 0, (hipStream_t)stream>>>(
                            (const T*)q, q_stride, (const T*)qnorm, eps, (const T*)gate, gate_stride, gate_w, (const T*)k_cache,
                            (const T*)v_cache, block_tables, bt_stride, block_size, cu_q, ctx0, tseq, H, G, d, dv, scale, window, chunk, rot_freq,
                            rot_dims, sink, qt_coef, qt_every, (T*)out));
  else                                               // heads of up to 1024 entries: the same kernel with 16 entries per lane
    NVS_DISPATCH(dtype, window_attn_kernel<T, 16><<<dim3((unsigned)n, H), dim3(64), 0, (hipStream_t)stream>>>(
                            (const T*)q, q_stride, (const T*)qnorm, eps, (const T*)gate, gate_stride, gate_w, (const T*)k_cache,
                            (const T*)v_cache, block_tables, bt_stride, block_size, cu_q, ctx0, tseq, H, G, d, dv, scale, window, chunk, rot_freq,
                            rot_dims, sink, qt_coef, qt_every, (T*)out));
  return nvs_check_launch("nvs_window_attn");
}
