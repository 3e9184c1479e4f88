// Stateful sequence kernels: causal convolution, real-gated linear recurrence, state-space-duality recurrence (recurrent
// form), gated group norm. State lives in 32-bit in per-sequence slots; a portion whose first token is position 0 starts
// from zeros whatever the slot holds.
#include "seq_common.h"
#include <stdlib.h>

namespace {

constexpr int MAX_TAPS = 16;

// ---- causal convolution -------------------------------------------------------------------------------------------
// one thread per (token, channel); inputs before the portion come from the slot's tail (or are zero at a sequence start)
template <typename T, typename TO>
__global__ void causal_conv_kernel(const T* __restrict__ in, int64_t in_stride, const T* __restrict__ w, const T* __restrict__ b,
                                   int channels, int taps, int act, const int32_t* __restrict__ cu_q,
                                   const int32_t* __restrict__ ctx0, const int32_t* __restrict__ slot,
                                   const int32_t* __restrict__ tseq, const float* __restrict__ state, TO* __restrict__ out,
                                   int64_t t0) {
  const int64_t t = t0 + blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int s = tseq[t];
  const int64_t q0 = cu_q[s];
  const int64_t rel = t - q0;                       // index inside the portion
  const bool fresh = ctx0[s] == 0;
  const float* tail = state + (int64_t)slot[s] * (taps - 1) * channels;
  float acc = b ? ldf(b + c) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int64_t back = (taps - 1) - j;            // tokens before the current one
    float v;
    if (rel >= back) {
      v = ldf(in + (t - back) * in_stride + c);
    } else if (fresh) {
      v = 0.f;
    } else {
      // tail[k] is the input (taps-1-k) tokens before the portion's first token; this tap looks (back - rel) before it
      const int k = (taps - 1) - (int)(back - rel);
      v = tail[(int64_t)k * channels + c];
    }
    acc += ldf(w + (int64_t)c * taps + j) * v;
  }
  if (act == 1) acc = siluf_(acc);
  stf(out + t * channels + c, acc);
}

// one thread per (portion, channel): the new tail is read completely before it is written
template <typename T>
__global__ void conv_state_kernel(const T* __restrict__ in, int64_t in_stride, int channels, int taps,
                                  const int32_t* __restrict__ cu_q, const int32_t* __restrict__ ctx0,
                                  const int32_t* __restrict__ slot, float* __restrict__ state) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int64_t q0 = cu_q[s], len = cu_q[s + 1] - q0;
  if (len <= 0) return;
  const bool fresh = ctx0[s] == 0;
  float* tail = state + (int64_t)slot[s] * (taps - 1) * channels;
  float nv[MAX_TAPS];
  for (int k = 0; k < taps - 1; ++k) {
    const int64_t back = (taps - 1) - k;            // new tail[k] = input `back` tokens before the END of the portion
    float v;
    if (len >= back) {
      v = ldf(in + (q0 + len - back) * in_stride + c);
    } else if (fresh) {
      v = 0.f;
    } else {
      v = tail[(int64_t)(k + len) * channels + c];  // the old tail, shifted by the portion's length
    }
    nv[k] = v;
  }
  for (int k = 0; k < taps - 1; ++k) tail[(int64_t)k * channels + c] = nv[k];
}

// ---- real-gated linear recurrence ---------------------------------------------------------------------------------
// One thread per (portion, channel), sequential over the portion's tokens; loads do not depend on the recurrence, so the
// compiler keeps several tokens' operands in flight. Long portions of a step with few (portion, channel) threads are cut
// into segments of seg_len tokens (blockIdx.z) and scanned twice, as the SSD scan below does:
//   mode 1: every segment but a portion's last from zero -> its final value L_k and decay product d_k to `ws`
//           ([nseq][nseg + 1][2][channels]; entry 0 holds the value the portion starts from);
//   mode 2: segment k starts from S_k = d_(k-1) S_(k-1) + L_(k-1) and writes the outputs; the last one writes the slot.
template <typename T, int MODE>
__global__ void rglru_scan_kernel(const float* __restrict__ gates, const float* __restrict__ u, const T* __restrict__ ypre,
                                  int64_t y_stride, const T* __restrict__ lam, float cmul, int channels, int blocks,
                                  const int32_t* __restrict__ cu_q, const int32_t* __restrict__ ctx0,
                                  const int32_t* __restrict__ slot, int64_t n, float* __restrict__ S, T* __restrict__ out, int seg_len,
                                  int nseg, float* __restrict__ ws) {
  constexpr int mode = MODE;                        // (compile-time: the plain scan keeps its straight-line loop)
  const int s = blockIdx.y, seg = blockIdx.z;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int64_t p0 = cu_q[s], p1 = cu_q[s + 1];
  const int64_t q0 = mode == 0 ? p0 : p0 + (int64_t)seg * seg_len;
  const int64_t q1 = mode == 0 ? p1 : (q0 + seg_len < p1 ? q0 + seg_len : p1);
  if (q1 <= q0) return;
  const bool last = q1 == p1;
  const int bw = channels / blocks, blk = c / bw, cc = c - blk * bw;
  const float sp = softplusf_(ldf(lam + c));
  float* sp_state = S + (int64_t)slot[s] * channels + c;
  float* wv = ws + ((int64_t)s * (nseg + 1)) * 2 * channels + c;          // entry e: value at + 2 e C, decay at + (2 e + 1) C
  float st = 0.f;
  if (mode == 2) {
    st = wv[0];
    for (int k = 0; k < seg; ++k) st = wv[(int64_t)(2 * k + 3) * channels] * st + wv[(int64_t)(2 * k + 2) * channels];
  } else if (ctx0[s] != 0 && (mode == 0 || seg == 0)) {
    st = *sp_state;
  }
  if (mode == 1) {
    if (seg == 0) wv[0] = st;
    if (last) return;
    st = 0.f;
  }
  float dsum = 0.f;                                 // sum of log a over the segment
  const float* gp = gates + ((int64_t)blk * n) * (2 * bw) + cc;
#pragma unroll 4
  for (int64_t t = q0; t < q1; ++t) {
    const float gr = gp[t * (2 * bw)], gi = gp[t * (2 * bw) + bw];
    const float uv = u[t * channels + c];
    const float r = 1.f / (1.f + expf(-gr)), ig = 1.f / (1.f + expf(-gi));
    const float log_a = -cmul * r * sp;
    const float a = expf(log_a);
    const float mult = sqrtf(fmaxf(-expm1f(2.f * log_a), 0.f));     // sqrt(1 - a^2), without cancellation near a = 1
    st = a * st + mult * (ig * uv);
    dsum += log_a;
    if (mode != 1) stf(out + t * channels + c, st * gelu_tanhf_(ldf(ypre + t * y_stride + c)));
  }
  if (mode == 1) {
    wv[(int64_t)(2 * seg + 2) * channels] = st;
    wv[(int64_t)(2 * seg + 3) * channels] = expf(dsum);
  } else if (last) {
    *sp_state = st;
  }
}

// Segments for the elementwise recurrence: seg_len 0 = none.
static void rglru_plan(int channels, int nseq, int64_t max_q, int* seg_len, int* nseg) {
  *seg_len = 0;
  *nseg = 1;
  const int64_t threads = (int64_t)channels * nseq;
  if (threads >= 131072 || max_q < 512) return;    // two wavefronts per SIMD already, or nothing to cut
  const int target = (int)((131072 + threads - 1) / threads);
  int64_t sl = (max_q + target - 1) / target;
  if (sl < 64) sl = 64;
  const int ns = (int)((max_q + sl - 1) / sl);
  if (ns < 2) return;
  *seg_len = (int)sl;
  *nseg = ns;
}

extern "C" int64_t nvs_rglru_scan_workspace(int channels, int nseq, int64_t max_q) {
  int seg_len, nseg;
  rglru_plan(channels, nseq, max_q, &seg_len, &nseg);
  return seg_len ? (int64_t)nseq * (nseg + 1) * 2 * channels : 0;
}

// ---- state-space-duality recurrence -------------------------------------------------------------------------------
// One workgroup per (portion, head), (P / PP) * NG threads: thread (tid / NG, g = tid % NG) keeps the 16 state entries
// S[p][16 g .. 16 g + 15] of PP consecutive p in registers (state memory is [heads][P][N], n fastest: a thread's entries are contiguous).
// Tokens go in rounds of TB: the round's x | B | C | dt | decay are staged in LDS by all threads, then every token costs 16 x (2 FMA + 1 MUL) per thread, LDS
// reads that vectorise, and log2(NG) shuffles for y[p] = sum_n S C: the NG threads of a p are neighbouring lanes.
constexpr int SSD_R = 16;      // state entries per thread
constexpr int SSD_TB = 16;     // tokens per LDS round
constexpr int SSD_SB = 8;      // tokens whose cross-lane sums are taken together

// FORM 0: the state-space-duality recurrence as described above. FORM 1: the decaying outer-product recurrence of linear
// ("lightning") attention, S <- decay_h S + k v^T, o = S^T q — the same walk with x = v, B = k, C = q, a step size of one, a
// decay that is a per-head constant (`decay`, 32-bit) and no skip term; v | k | q are read from the projection output itself
// (columns x_col / b_col / c_col + the head's offset, `dtype`) and SiLU is applied as they are staged.
// FORM 2: the matrix memory with exponential gates. Per head and token, from the gate pre-activations zi, zf (columns i_col / f_col
// + head of the projection output, plus a bias each): i = cap tanh(zi / cap), f = logsigmoid(cap tanh(zf / cap)); with a running
// maximum m (0 at a sequence's start) m' = max(f + m, i), S <- exp(f + m - m') S + exp(i - m') k v^T, n likewise with k alone. The
// walk is the same with x = v, B = k, C = q * c_scale, decay exp(f + m - m'), step exp(i - m') — per round of tokens the gates are
// computed a token per thread, ONE thread walks the maximum through them, and the exponentials are again a token per thread —
// and n is simply one more row of the state, whose "value" is
// the constant 1: the kernel sees P = dv + 1 rows (state memory [heads][dv + 1][dk], M [nslots][heads] holds m). It writes the
// numerators S^T q to y [n, heads * dv] and den [n, heads] = max(|n . q|, exp(-m')) + 1e-6; the division is left to the norm that
// follows. Segments: a segment scanned from nothing (its own maximum starting at "minus infinity") ends with a local state L, a
// local maximum ml and the sum F of its log forget gates; behind a state (S, m) the true state after it is m' = max(m + F, ml),
// S' = exp(m + F - m') S + exp(ml - m') L — the same sum of terms, scaled by another maximum — so mode 2 combines the segments
// before its own in order and then walks its tokens as usual (`ws` holds F and ml beside every local state).
template <typename T, int PP, int MODE, int FORM = 0>     // PP head-size entries per thread: the B / C values read from LDS serve PP state rows
__global__ __launch_bounds__(FORM == 2 ? (PP == 4 ? 512 : (PP == 2 ? 576 : 1024)) : (PP == 4 ? 256 : (PP == 2 ? 512 : 1024))) void ssd_scan_kernel(const float* __restrict__ xbc, const T* __restrict__ proj, int64_t proj_stride, int64_t dt_col,
                                int64_t x_col, int64_t b_col, int64_t c_col, const float* __restrict__ decay,
                                const T* __restrict__ dt_bias, const T* __restrict__ A_log, const T* __restrict__ Dp, int heads,
                                int P, int N, int G, int NG, int TB, const int32_t* __restrict__ cu_q,
                                const int32_t* __restrict__ ctx0, const int32_t* __restrict__ slot, float* __restrict__ S,
                                float* __restrict__ y, int seg_len, int nseg, float* __restrict__ ws, int64_t i_col, int64_t f_col,
                                const T* __restrict__ i_bias, const T* __restrict__ f_bias, float cap, float c_scale,
                                float* __restrict__ M, float* __restrict__ den) {
  constexpr int mode = MODE;                        // (compile-time: the unsegmented scan pays nothing for the other two)
  // mode 0: the whole portion in one workgroup. Long portions with few (portion, head) pairs are cut into segments of
  // seg_len tokens (blockIdx.z) and scanned twice, because one workgroup walks its tokens one after the other:
  //   mode 1: every segment but a portion's last from a ZERO state -> its final state L_k and decay product d_k to `ws`
  //           (entry 0 of a (portion, head) holds the state the portion starts from);
  //   mode 2: segment k starts from S_k = d_(k-1) S_(k-1) + L_(k-1), S_0 = entry 0, and produces y; the last one writes the slot.
  extern __shared__ __attribute__((aligned(16))) float lds[];   // [TB][per]: x (P) | B (NP) | C (NP) | dt, NP = 16 NG, zero padded
  const int s = blockIdx.y, h = blockIdx.x, tid = threadIdx.x, nthreads = blockDim.x;
  const int g = tid & (NG - 1), p = (tid / NG) * PP;          // this thread's first p
  const int64_t p0 = cu_q[s], p1 = cu_q[s + 1];
  const int seg = blockIdx.z;
  const int64_t q0 = mode == 0 ? p0 : p0 + (int64_t)seg * seg_len;
  const int64_t q1 = mode == 0 ? p1 : (q0 + seg_len < p1 ? q0 + seg_len : p1);
  if (q1 <= q0) return;
  const bool last = q1 == p1;
  if (mode == 1 && last && seg > 0) return;         // nobody starts from the last segment's state
  float* wst = ws + ((int64_t)(s * heads + h) * (nseg + 1)) * P * N + (int64_t)p * N + g * SSD_R;   // entry e: + e P N
  constexpr int WD = FORM == 2 ? 3 : 1;             // numbers kept beside a segment's state: its decay product, or F and ml
  float* wdec = ws + (int64_t)gridDim.y * heads * (nseg + 1) * P * N + (int64_t)(s * heads + h) * (nseg + 1) * WD;
  // every part starts 16-byte aligned; the x part also covers the rows of the last thread that lie beyond P (zeros: form 2's row count need not divide)
  const int NP = NG * SSD_R, P4 = ((P + PP - 1) / PP * PP + 3) & ~3, per = P4 + 2 * NP + 4;
  const int inner = heads * P, grp = h / (heads / G);
  const int64_t row = inner + 2 * G * N;
  float A = 0.f, Dh = 0.f, dtb = 0.f, fixed_decay = 1.f;
  if (FORM == 0) {
    A = -expf(ldf(A_log + h)), Dh = ldf(Dp + h), dtb = ldf(dt_bias + h);
  } else {
    fixed_decay = decay[h];
  }
  float* Sh = S + (((int64_t)slot[s] * heads + h) * P + p) * N + g * SSD_R;
  float st[PP][SSD_R];
  const bool fresh = ctx0[s] == 0;
  // FORM 2: the running maximum (kept by the one thread that turns gates into decays), the gates' biases, rows beyond P are idle
  const int Py = FORM == 2 ? P - 1 : P;             // rows that are outputs
  float mrun = 0.f, bi = 0.f, bf = 0.f, fsum = 0.f;
  if (FORM == 2) {
    bi = ldf(i_bias + h), bf = ldf(f_bias + h);
    if (!fresh) mrun = M[(int64_t)slot[s] * heads + h];
    if (mode == 1) {                                // the portion's starting maximum for mode 2; a segment by itself starts from none
      if (seg == 0 && tid == 0) wdec[1] = mrun;
      mrun = -1e30f;
    }
    if (mode == 2) mrun = wdec[1];
  }
  const bool vec = (N & 3) == 0;                    // a thread's 16 entries are then four aligned 16-byte pieces
  auto load16 = [&](const float* src, float (&dst)[SSD_R]) {
    if (vec) {
#pragma unroll
      for (int r = 0; r < SSD_R; r += 4) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (g * SSD_R + r < N) v = *(const float4*)(src + r);
        dst[r] = v.x, dst[r + 1] = v.y, dst[r + 2] = v.z, dst[r + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int r = 0; r < SSD_R; ++r) dst[r] = g * SSD_R + r < N ? src[r] : 0.f;
    }
  };
  auto store16 = [&](float* dst, const float (&src)[SSD_R]) {
    if (vec) {
#pragma unroll
      for (int r = 0; r < SSD_R; r += 4)
        if (g * SSD_R + r < N) *(float4*)(dst + r) = make_float4(src[r], src[r + 1], src[r + 2], src[r + 3]);
    } else {
#pragma unroll
      for (int r = 0; r < SSD_R; ++r)
        if (g * SSD_R + r < N) dst[r] = src[r];
    }
  };
#pragma unroll
  for (int i = 0; i < PP; ++i) {
#pragma unroll
    for (int r = 0; r < SSD_R; ++r) st[i][r] = 0.f;
    const bool row_ok = FORM != 2 || p + i < P;     // (form 2's last thread may hold rows beyond the state)
    if (mode == 2) {
      if (row_ok) load16(wst + (int64_t)i * N, st[i]);          // S_0, then the segments before this one
      float mk = FORM == 2 ? wdec[1] : 0.f;
      for (int k = 0; k < seg; ++k) {
        float lk[SSD_R];
#pragma unroll
        for (int r = 0; r < SSD_R; ++r) lk[r] = 0.f;
        if (row_ok) load16(wst + (int64_t)(k + 1) * P * N + (int64_t)i * N, lk);
        float dk = wdec[(k + 1) * WD], bk = 1.f;
        if (FORM == 2) {
          const float F = wdec[(k + 1) * WD], ml = wdec[(k + 1) * WD + 1];
          const float mn = fmaxf(mk + F, ml);
          dk = expf(mk + F - mn), bk = expf(ml - mn);
          mk = mn;
        }
#pragma unroll
        for (int r = 0; r < SSD_R; ++r) st[i][r] = dk * st[i][r] + bk * lk[r];
      }
      if (FORM == 2) mrun = mk;
    } else if (!fresh && (mode == 0 || seg == 0) && (FORM != 2 || p + i < P)) {
      load16(Sh + (int64_t)i * N, st[i]);
    }
    if (mode == 1 && seg == 0) {                    // the portion's starting state, for mode 2
      if (row_ok) store16(wst + (int64_t)i * N, st[i]);
#pragma unroll
      for (int r = 0; r < SSD_R; ++r) st[i][r] = 0.f;
    }
  }
  if (mode == 1 && last) return;                    // (a portion of one segment: only its starting state was needed)
  float dprod = 1.f;

  const float* xh = xbc + h * P;
  float* yh = y + h * Py + p;
  const int inner_y = heads * Py;
  const float* Bg = xbc + inner + grp * N;
  const float* Cg = Bg + G * N;
  const T* xh1 = proj + x_col + h * Py;             // FORM 1, 2: the three operands inside the projection output
  const T* Bg1 = proj + b_col + grp * N;
  const T* Cg1 = proj + c_col + grp * N;
  for (int64_t tb = q0; tb < q1; tb += TB) {
    const int cnt = (int)((q1 - tb) < TB ? (q1 - tb) : TB);
    __syncthreads();                                // the previous round's readers are done
    // stage the round: other workgroups of the CU compute meanwhile (LDS and registers leave room for several)
    // a thread stages ONE column of the image for all tokens of the round: the column is classified once, the 16 loads are
    // independent and in flight together, and for a fixed token neighbouring threads read neighbouring addresses
    for (int c = tid; c < per; c += nthreads) {
      const float* src = nullptr;                   // a 32-bit source with row stride `row`
      const T* src1 = nullptr;                      // FORM 1: a source in the projection output, SiLU applied here
      int kind = 0;                                 // 0: padding (zero), 1: x / B / C, 2: step size, 3: decay
      if (FORM == 2 && c == P - 1) {
        kind = 4;                                   // the normaliser's row: its "value" is the constant 1
      } else if (c < P) {
        src = xh + c, src1 = xh1 + c, kind = 1;
      } else if (c >= P4 && c < P4 + NP) {
        if (c - P4 < N) src = Bg + (c - P4), src1 = Bg1 + (c - P4), kind = 1;
      } else if (c >= P4 + NP && c < P4 + 2 * NP) {
        if (c - P4 - NP < N) src = Cg + (c - P4 - NP), src1 = Cg1 + (c - P4 - NP), kind = FORM == 2 ? 5 : 1;
      } else if (c == P4 + 2 * NP) {
        kind = 2;
      } else if (c == P4 + 2 * NP + 1) {
        kind = 3;
      }
      float v[SSD_TB];
      if (FORM == 2 && c >= P4 + 2 * NP) continue;  // (step, decay, exp(-m): from the gates, below)
#pragma unroll
      for (int k = 0; k < SSD_TB; ++k) {
        v[k] = 0.f;
        if (k < cnt) {
          if (FORM == 0) {
            if (kind == 1) v[k] = src[(tb + k) * row];
            if (kind >= 2) v[k] = ldf(proj + (tb + k) * proj_stride + dt_col + h);
          } else {
            if (kind == 1 || kind == 5) v[k] = ldf(src1 + (tb + k) * proj_stride);
          }
        }
      }
#pragma unroll
      for (int k = 0; k < SSD_TB; ++k) {
        if (k < cnt) {
          float w = v[k];
          if (FORM == 0) {
            if (kind >= 2) {
              w = softplusf_(w + dtb);
              if (kind == 3) w = expf(A * w);
            }
          } else if (FORM == 1) {
            if (kind == 1) w = siluf_(w);
            if (kind == 2) w = 1.f;
            if (kind == 3) w = fixed_decay;
          } else {
            if (kind == 4) w = 1.f;
            if (kind == 5) w *= c_scale;
          }
          lds[k * per + c] = w;
        }
      }
    }
    float* gates = lds + P4 + 2 * NP;               // FORM 2: per token (+ k * per) the gates i, f -> step, decay, exp(-m)
    if (FORM == 2) {
      for (int k = tid; k < cnt; k += nthreads) {   // the gates themselves, a token per thread
        const float zi = ldf(proj + (tb + k) * proj_stride + i_col + h), zf = ldf(proj + (tb + k) * proj_stride + f_col + h);
        const float zc = cap * tanhf((zf + bf) / cap);
        gates[k * per] = cap * tanhf((zi + bi) / cap);
        gates[k * per + 1] = fminf(zc, 0.f) - log1pf(expf(-fabsf(zc)));          // log sigmoid
      }
    }
    __syncthreads();
    if (FORM == 2) {
      if (tid == 0) {                               // the running maximum, token after token: an add and a max each
        for (int k = 0; k < cnt; ++k) {
          const float mn = fmaxf(gates[k * per + 1] + mrun, gates[k * per]);
          gates[k * per + 2] = mrun;
          gates[k * per + 3] = mn;
          fsum += gates[k * per + 1];
          mrun = mn;
        }
      }
      __syncthreads();
      for (int k = tid; k < cnt; k += nthreads) {
        const float gi = gates[k * per], gf = gates[k * per + 1], mb = gates[k * per + 2], mn = gates[k * per + 3];
        gates[k * per] = expf(gi - mn);
        gates[k * per + 1] = expf(gf + mb - mn);
        gates[k * per + 2] = expf(-mn);
      }
      __syncthreads();
    }
    // one token: S <- dA S + dt B x; returns this thread's share of y = S . C for each of its rows
    auto token = [&](int k, float (&part)[PP], float (&xs)[PP]) {
      const float* tp = lds + k * per;
      const float dt = tp[P4 + 2 * NP], dA = tp[P4 + 2 * NP + 1];
      dprod *= dA;
      const float* Bp = (const float*)__builtin_assume_aligned(tp + P4 + g * SSD_R, 16);
      const float* Cp = (const float*)__builtin_assume_aligned(Bp + NP, 16);
      float bv[SSD_R], cv[SSD_R];
#pragma unroll
      for (int r = 0; r < SSD_R; ++r) bv[r] = Bp[r], cv[r] = Cp[r];
#pragma unroll
      for (int i = 0; i < PP; ++i) {
        const float xv = tp[p + i];
        const float dx = dt * xv;
        float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
        for (int r = 0; r < SSD_R; r += 2) {
          st[i][r] = dA * st[i][r] + bv[r] * dx;
          st[i][r + 1] = dA * st[i][r + 1] + bv[r + 1] * dx;
          acc0 += st[i][r] * cv[r];
          acc1 += st[i][r + 1] * cv[r + 1];
        }
        part[i] = acc0 + acc1;
        xs[i] = xv;
      }
    };
    if (cnt == SSD_TB) {
      // a full round: the cross-lane sums of all its tokens are taken together AFTER the token loop — a shuffle per token
      // would put a wait for every outstanding LDS access into each step of the recurrence
#pragma unroll 1
      for (int k0 = 0; k0 < SSD_TB; k0 += SSD_SB) {
        float part[SSD_SB][PP], xs[SSD_SB][PP];
#pragma unroll
        for (int k = 0; k < SSD_SB; ++k) token(k0 + k, part[k], xs[k]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
          if (o < NG) {
#pragma unroll
            for (int k = 0; k < SSD_SB; ++k)
#pragma unroll
              for (int i = 0; i < PP; ++i) part[k][i] += __shfl_xor(part[k][i], o, 64);
          }
        }
        if (g == 0 && mode != 1) {
#pragma unroll
          for (int k = 0; k < SSD_SB; ++k)
#pragma unroll
            for (int i = 0; i < PP; ++i) {
              if (FORM == 2) {
                if (p + i < Py) yh[(tb + k0 + k) * inner_y + i] = part[k][i];
                else if (p + i == Py) den[(tb + k0 + k) * heads + h] = fmaxf(fabsf(part[k][i]), lds[(k0 + k) * per + P4 + 2 * NP + 2]) + 1e-6f;
              } else {
                yh[(tb + k0 + k) * inner + i] = part[k][i] + Dh * xs[k][i];
              }
            }
        }
      }
    } else {
      for (int k = 0; k < cnt; ++k) {
        float part[PP], xs[PP];
        token(k, part, xs);
#pragma unroll
        for (int i = 0; i < PP; ++i) {
          float acc = part[i];
          for (int o = NG >> 1; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
          if (g == 0 && mode != 1) {
            if (FORM == 2) {
              if (p + i < Py) yh[(tb + k) * inner_y + i] = acc;
              else if (p + i == Py) den[(tb + k) * heads + h] = fmaxf(fabsf(acc), lds[k * per + P4 + 2 * NP + 2]) + 1e-6f;
            } else {
              yh[(tb + k) * inner + i] = acc + Dh * xs[i];
            }
          }
        }
      }
    }
  }
  if (mode == 1) {
#pragma unroll
    for (int i = 0; i < PP; ++i)
      if (FORM != 2 || p + i < P) store16(wst + (int64_t)(seg + 1) * P * N + (int64_t)i * N, st[i]);
    if (tid == 0) {
      if (FORM == 2) wdec[(seg + 1) * WD] = fsum, wdec[(seg + 1) * WD + 1] = mrun;
      else wdec[seg + 1] = dprod;
    }
  } else if (last) {
#pragma unroll
    for (int i = 0; i < PP; ++i)
      if (FORM != 2 || p + i < P) store16(Sh + (int64_t)i * N, st[i]);
    if (FORM == 2 && tid == 0) M[(int64_t)slot[s] * heads + h] = mrun;      // the thread that kept it
  }
}

// ---- gate, then group RMS norm ------------------------------------------------------------------------------------
// one workgroup per (token, group)
template <typename T>
__global__ void gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ z, int64_t z_stride,
                                        const T* __restrict__ w, int inner, int groups, float eps, int order,
                                        const float* __restrict__ den, T* __restrict__ out) {
  __shared__ float red[16];
  const int64_t t = blockIdx.y;
  const int gsz = inner / groups, c0 = blockIdx.x * gsz;
  float ss = 0.f;
  if (order == 1) {                                 // norm first, then a sigmoid gate
    const float dinv = den ? 1.f / den[t * groups + blockIdx.x] : 1.f;      // the group's entries are numerators over this
    for (int c = threadIdx.x; c < gsz; c += blockDim.x) {
      const float v = y[t * inner + c0 + c] * dinv;
      ss += v * v;
    }
    const float r = 1.f / sqrtf(block_sum(ss, red) / (float)gsz + eps);
    for (int c = threadIdx.x; c < gsz; c += blockDim.x) {
      const float gz = ldf(z + t * z_stride + c0 + c);
      stf(out + t * inner + c0 + c, y[t * inner + c0 + c] * dinv * r * ldf(w + c0 + c) * (1.f / (1.f + expf(-gz))));
    }
    return;
  }
  for (int c = threadIdx.x; c < gsz; c += blockDim.x) {
    const float v = y[t * inner + c0 + c] * siluf_(ldf(z + t * z_stride + c0 + c));
    ss += v * v;
  }
  const float r = rsqrtf(block_sum(ss, red) / (float)gsz + eps);
  for (int c = threadIdx.x; c < gsz; c += blockDim.x) {
    const float v = y[t * inner + c0 + c] * siluf_(ldf(z + t * z_stride + c0 + c));
    stf(out + t * inner + c0 + c, v * r * ldf(w + c0 + c));
  }
}

}  // namespace

extern "C" int nvs_causal_conv(const void* in, int64_t in_stride, int dtype, const void* w, const void* b, int channels, int taps,
                               int act, const int32_t* cu_q, const int32_t* ctx0, const int32_t* slot, const int32_t* tseq, int nseq,
                               int64_t n, float* state, void* out, int out_dtype, void* stream) {
  NVS_REQUIRE(out_dtype == NVS_F32 || out_dtype == dtype, "nvs_causal_conv: the output is 32-bit or of the input's type");
  NVS_REQUIRE(in && w && cu_q && ctx0 && slot && tseq && (state || taps == 1) && out, "nvs_causal_conv: null argument");
  NVS_REQUIRE(channels > 0 && taps >= 1 && taps <= MAX_TAPS && in_stride >= channels && nseq >= 0 && n >= 0 && (act == 0 || act == 1),
              "nvs_causal_conv: channels %d taps %d (1..%d) stride %lld act %d", channels, taps, MAX_TAPS, (long long)in_stride, act);
  if (n == 0 || nseq == 0) return NVS_OK;
  NVS_REQUIRE(n <= 65535 * 64ll && nseq <= 65535, "nvs_causal_conv: step too large");
  const dim3 block(channels >= 256 ? 256 : 64);
  const unsigned gx = (channels + block.x - 1) / block.x;
  // grid.y is limited to 65535: larger steps go in slices
  for (int64_t t0 = 0; t0 < n; t0 += 65535) {
    const int64_t cnt = n - t0 < 65535 ? n - t0 : 65535;
    if (out_dtype == NVS_F32)
      NVS_DISPATCH(dtype, causal_conv_kernel<T, float><<<dim3(gx, (unsigned)cnt), block, 0, (hipStream_t)stream>>>(
                              (const T*)in, in_stride, (const T*)w, (const T*)b, channels, taps, act, cu_q, ctx0, slot, tseq, state,
                              (float*)out, t0));
    else
      NVS_DISPATCH(dtype, causal_conv_kernel<T, T><<<dim3(gx, (unsigned)cnt), block, 0, (hipStream_t)stream>>>(
                              (const T*)in, in_stride, (const T*)w, (const T*)b, channels, taps, act, cu_q, ctx0, slot, tseq, state,
                              (T*)out, t0));
  }
  int rc = nvs_check_launch("nvs_causal_conv");
  if (rc) return rc;
  if (taps > 1) {
    NVS_DISPATCH(dtype, conv_state_kernel<T><<<dim3(gx, (unsigned)nseq), block, 0, (hipStream_t)stream>>>(
                            (const T*)in, in_stride, channels, taps, cu_q, ctx0, slot, state));
    rc = nvs_check_launch("nvs_causal_conv (state)");
  }
  return rc;
}

extern "C" int nvs_rglru_scan(const float* gates, const float* u, const void* ypre, int64_t y_stride, int dtype, const void* lam,
                              float c, int channels, int blocks, const int32_t* cu_q, const int32_t* ctx0, const int32_t* slot, int nseq,
                              int64_t n, int64_t max_q, float* S, void* out, float* ws, int64_t ws_floats, void* stream) {
  NVS_REQUIRE(gates && u && ypre && lam && cu_q && ctx0 && slot && S && out, "nvs_rglru_scan: null argument");
  NVS_REQUIRE(channels > 0 && blocks > 0 && channels % blocks == 0 && y_stride >= channels && nseq >= 0 && nseq <= 65535 && n >= 0,
              "nvs_rglru_scan: channels %d blocks %d", channels, blocks);
  if (n == 0 || nseq == 0) return NVS_OK;
  int seg_len = 0, nseg = 1;
  if (ws) rglru_plan(channels, nseq, max_q > 0 ? max_q : n, &seg_len, &nseg);
  NVS_REQUIRE(!seg_len || ws_floats >= nvs_rglru_scan_workspace(channels, nseq, max_q > 0 ? max_q : n),
              "nvs_rglru_scan: workspace of %lld floats is too small", (long long)ws_floats);
  const dim3 block(64);
#define NVS_RGLRU_LAUNCH(MODE)                                                                                                     \
  NVS_DISPATCH(dtype, rglru_scan_kernel<T, MODE><<<dim3((channels + 63) / 64, (unsigned)nseq, seg_len ? nseg : 1), block, 0,         \
                                                  (hipStream_t)stream>>>(gates, u, (const T*)ypre, y_stride, (const T*)lam, c, channels, \
                                                                         blocks, cu_q, ctx0, slot, n, S, (T*)out, seg_len, nseg, ws))
  if (seg_len) {
    NVS_RGLRU_LAUNCH(1);
    NVS_RGLRU_LAUNCH(2);
  } else {
    NVS_RGLRU_LAUNCH(0);
  }
#undef NVS_RGLRU_LAUNCH
  return nvs_check_launch("nvs_rglru_scan");
}

// Segments for long portions when (portion, head) pairs alone would leave compute units idle: seg_len 0 = none.
static void ssd_plan(int heads, int nseq, int64_t max_q, int* seg_len, int* nseg, int full_at = 512) {
  *seg_len = 0;
  *nseg = 1;
  const int64_t pairs = (int64_t)heads * nseq;
  // (measured, 8 x 2048 tokens: 128 pairs 11.8 ms per step unsegmented -> 9.8 with 1,024 workgroups -> 9.3 with 2,048; 512 pairs,
  //  two workgroups per CU already, LOSE with two or four segments each: 18.7 -> 19.8 - 20.0)
  // (the matrix memory's workgroups are larger — one per compute unit — and 256 pairs already lose: 8 x 2048 tokens x 32 heads of
  //  128 x 128 take 3.9 ms in one pass, 2.0 + 3.9 ms in segments; 64 pairs 3.85 ms against 0.45 + 0.95; it passes full_at = 192)
  if (pairs >= full_at || max_q < 512) return;
  const int target = (int)((2048 + pairs - 1) / pairs);     // segments wanted per portion
  int64_t sl = (max_q + target - 1) / target;
  sl = (sl + 15) / 16 * 16;
  if (sl < 128) sl = 128;
  const int ns = (int)((max_q + sl - 1) / sl);
  if (ns < 2) return;
  *seg_len = (int)sl;
  *nseg = ns;
}

extern "C" int64_t nvs_ssd_scan_workspace(int heads, int P, int N, int nseq, int64_t max_q) {
  int seg_len, nseg;
  ssd_plan(heads, nseq, max_q, &seg_len, &nseg);
  return seg_len ? (int64_t)nseq * heads * (nseg + 1) * ((int64_t)P * N + 1) : 0;
}

extern "C" int64_t nvs_gated_memory_scan_workspace(int heads, int dk, int dv, int nseq, int64_t max_q) {
  int seg_len, nseg;
  ssd_plan(heads, nseq, max_q, &seg_len, &nseg, 192);
  return seg_len ? (int64_t)nseq * heads * (nseg + 1) * ((int64_t)(dv + 1) * dk + 3) : 0;
}

// what only the matrix memory (form 2) passes
struct GateArgs {
  int64_t i_col = 0, f_col = 0;
  const void *i_bias = nullptr, *f_bias = nullptr;
  float cap = 0.f, c_scale = 1.f;
  float *M = nullptr, *den = nullptr;
};

// all forms of the scan: argument checks that they share, the plan, the launches
static int ssd_launch(int form, const char* who, const float* xbc, const void* proj, int64_t proj_stride, int64_t dt_col, int64_t x_col,
                      int64_t b_col, int64_t c_col, const float* decay, int dtype, const void* dt_bias, const void* A_log, const void* D,
                      int heads, int P, int N, int G, const int32_t* cu_q, const int32_t* ctx0, const int32_t* slot, int nseq, int64_t n,
                      int64_t max_q, float* S, float* y, float* ws, int64_t ws_floats, void* stream, const GateArgs& ga = GateArgs()) {
  NVS_REQUIRE(heads > 0 && G > 0 && heads % G == 0 && P > 0 && P <= 257 && N > 0 && nseq >= 0 && nseq <= 65535,
              "%s: heads %d groups %d head size %d state %d", who, heads, G, P, N);
  if (n == 0 || nseq == 0) return NVS_OK;
  int ng = 1;
  while (ng * SSD_R < N) ng <<= 1;                  // a power of two: the threads of one p reduce by lane shuffles
  const int ng0 = ng;
  // Rows per thread: the 32 B / C values a thread reads from LDS per token serve PP rows, and the scan is bound by the LDS
  // pipe at PP = 1 (counters: 21 LDS instructions against 93 VALU per wavefront and token, 8 of them 16-byte reads). PP = 4
  // leaves one wavefront per SIMD and is latency-bound instead (measured slower); PP = 2 is the default where it fits.
  // NVS_SSD_PP = 1 / 2 / 4 overrides for measurements.
  static const int forced = getenv("NVS_SSD_PP") ? atoi(getenv("NVS_SSD_PP")) : 0;
  int pp = forced ? forced : 2;
  if (form == 2) {                                  // (rows need not divide: the kernel guards them; one row more than outputs)
    if (((P + 1) / 2) * ng0 > 576) pp = ((P + 3) / 4) * ng0 <= 512 ? 4 : 1;
  } else {
    while (pp > 1 && (P % pp != 0 || (P / pp) * ng0 > (pp == 4 ? 256 : 512))) pp >>= 1;
  }
  NVS_REQUIRE(ng <= 64 && (int64_t)((P + pp - 1) / pp) * ng <= 1024, "%s: state %d x head size %d exceeds one workgroup's registers", who, N, P);
  const int threads = ((P + pp - 1) / pp) * ng, per = (((P + pp - 1) / pp * pp + 3) & ~3) + 2 * ng * SSD_R + 4;
  const int tb = SSD_TB;                            // tokens per LDS round
  const size_t lds = (size_t)tb * per * sizeof(float);
  int seg_len = 0, nseg = 1;
  if (ws) ssd_plan(heads, nseq, max_q > 0 ? max_q : n, &seg_len, &nseg, form == 2 ? 192 : 512);
  NVS_REQUIRE(!seg_len || ws_floats >= (form == 2 ? nvs_gated_memory_scan_workspace(heads, N, P - 1, nseq, max_q > 0 ? max_q : n)
                                                   : nvs_ssd_scan_workspace(heads, P, N, nseq, max_q > 0 ? max_q : n)),
              "%s: workspace of %lld floats is too small", who, (long long)ws_floats);
  const dim3 grid(heads, (unsigned)nseq, seg_len ? nseg : 1);
#define NVS_SSD_LAUNCH(PPV, MODE, FORM)                                                                                             \
  NVS_DISPATCH(dtype, ssd_scan_kernel<T, PPV, MODE, FORM><<<grid, dim3(threads), lds, (hipStream_t)stream>>>(                        \
                          xbc, (const T*)proj, proj_stride, dt_col, x_col, b_col, c_col, decay, (const T*)dt_bias, (const T*)A_log,   \
                          (const T*)D, heads, P, N, G, ng, tb, cu_q, ctx0, slot, S, y, seg_len, nseg, ws, ga.i_col, ga.f_col,                \
                          (const T*)ga.i_bias, (const T*)ga.f_bias, ga.cap, ga.c_scale, ga.M, ga.den))
#define NVS_SSD_PASSES(PPV, FORM)   \
  if (seg_len) {                    \
    NVS_SSD_LAUNCH(PPV, 1, FORM);   \
    NVS_SSD_LAUNCH(PPV, 2, FORM);   \
  } else {                          \
    NVS_SSD_LAUNCH(PPV, 0, FORM);   \
  }
#define NVS_SSD_FORMS(PPV)        \
  if (form == 0) {                \
    NVS_SSD_PASSES(PPV, 0)        \
  } else if (form == 1) {         \
    NVS_SSD_PASSES(PPV, 1)        \
  } else {                        \
    NVS_SSD_PASSES(PPV, 2)        \
  }
  if (pp == 2) {
    NVS_SSD_FORMS(2)
  } else if (pp == 4) {
    NVS_SSD_FORMS(4)
  } else {
    NVS_SSD_FORMS(1)
  }
#undef NVS_SSD_FORMS
#undef NVS_SSD_PASSES
#undef NVS_SSD_LAUNCH
  return nvs_check_launch(who);
}

extern "C" int nvs_ssd_scan(const float* xbc, const void* proj, int64_t proj_stride, int64_t dt_col, int dtype, const void* dt_bias,
                            const void* A_log, const void* D, int heads, int P, int N, int G, const int32_t* cu_q, const int32_t* ctx0,
                            const int32_t* slot, int nseq, int64_t n, int64_t max_q, float* S, float* y, float* ws, int64_t ws_floats,
                            void* stream) {
  NVS_REQUIRE(xbc && proj && dt_bias && A_log && D && cu_q && ctx0 && slot && S && y, "nvs_ssd_scan: null argument");
  return ssd_launch(0, "nvs_ssd_scan", xbc, proj, proj_stride, dt_col, 0, 0, 0, nullptr, dtype, dt_bias, A_log, D, heads, P, N, G, cu_q,
                    ctx0, slot, nseq, n, max_q, S, y, ws, ws_floats, stream);
}

extern "C" int nvs_decay_scan(const void* proj, int64_t proj_stride, int64_t v_col, int64_t k_col, int64_t q_col, int dtype,
                              const float* decay, int heads, int dk, int dv, const int32_t* cu_q, const int32_t* ctx0,
                              const int32_t* slot, int nseq, int64_t n, int64_t max_q, float* S, float* y, float* ws, int64_t ws_floats,
                              void* stream) {
  NVS_REQUIRE(proj && decay && cu_q && ctx0 && slot && S && y, "nvs_decay_scan: null argument");
  NVS_REQUIRE(v_col >= 0 && k_col >= 0 && q_col >= 0 && v_col + (int64_t)heads * dv <= proj_stride &&
                  k_col + (int64_t)heads * dk <= proj_stride && q_col + (int64_t)heads * dk <= proj_stride,
              "nvs_decay_scan: columns beyond the row stride %lld", (long long)proj_stride);
  return ssd_launch(1, "nvs_decay_scan", nullptr, proj, proj_stride, 0, v_col, k_col, q_col, decay, dtype, nullptr, nullptr, nullptr, heads,
                    dv, dk, heads, cu_q, ctx0, slot, nseq, n, max_q, S, y, ws, ws_floats, stream);
}

extern "C" int nvs_gated_memory_scan(const void* proj, int64_t proj_stride, int64_t v_col, int64_t k_col, int64_t q_col, int64_t i_col,
                                     int64_t f_col, int dtype, const void* i_bias, const void* f_bias, float cap, float q_scale, int heads,
                                     int dk, int dv, const int32_t* cu_q, const int32_t* ctx0, const int32_t* slot, int nseq, int64_t n,
                                     int64_t max_q, float* S, float* M, float* y, float* den, float* ws, int64_t ws_floats, void* stream) {
  NVS_REQUIRE(proj && i_bias && f_bias && cu_q && ctx0 && slot && S && M && y && den, "nvs_gated_memory_scan: null argument");
  NVS_REQUIRE(cap > 0.f && dv > 0 && dv <= 256, "nvs_gated_memory_scan: cap %g, value size %d", (double)cap, dv);
  NVS_REQUIRE(v_col >= 0 && k_col >= 0 && q_col >= 0 && i_col >= 0 && f_col >= 0 && v_col + (int64_t)heads * dv <= proj_stride &&
                  k_col + (int64_t)heads * dk <= proj_stride && q_col + (int64_t)heads * dk <= proj_stride &&
                  i_col + heads <= proj_stride && f_col + heads <= proj_stride,
              "nvs_gated_memory_scan: columns beyond the row stride %lld", (long long)proj_stride);
  GateArgs ga;
  ga.i_col = i_col, ga.f_col = f_col, ga.i_bias = i_bias, ga.f_bias = f_bias, ga.cap = cap, ga.c_scale = q_scale, ga.M = M, ga.den = den;
  return ssd_launch(2, "nvs_gated_memory_scan", nullptr, proj, proj_stride, 0, v_col, k_col, q_col, nullptr, dtype, nullptr, nullptr, nullptr,
                    heads, dv + 1, dk, heads, cu_q, ctx0, slot, nseq, n, max_q, S, y, ws, ws_floats, stream, ga);
}

extern "C" int nvs_gated_group_norm(const float* y, const void* z, int64_t z_stride, int dtype, const void* w, int inner, int groups,
                                    float eps, int order, int64_t n, const float* den, void* out, void* stream) {
  NVS_REQUIRE(!den || order == 1, "nvs_gated_group_norm: a divisor goes with the order norm, then gate");
  NVS_REQUIRE(y && z && w && out && inner > 0 && groups > 0 && inner % groups == 0 && z_stride >= inner && n >= 0 &&
                  (order == 0 || order == 1),
              "nvs_gated_group_norm: inner %d groups %d order %d", inner, groups, order);
  if (n == 0) return NVS_OK;
  NVS_REQUIRE(n <= 65535ll * 65535ll, "nvs_gated_group_norm: step too large");
  const int gsz = inner / groups;
  const dim3 block(gsz >= 1024 ? 256 : (gsz >= 128 ? 128 : 64));
  for (int64_t t0 = 0; t0 < n; t0 += 65535) {
    const int64_t cnt = n - t0 < 65535 ? n - t0 : 65535;
    NVS_DISPATCH(dtype, gated_group_norm_kernel<T><<<dim3(groups, (unsigned)cnt), block, 0, (hipStream_t)stream>>>(
                            y + t0 * inner, (const T*)z + t0 * z_stride, z_stride, (const T*)w, inner, groups, eps, order,
                            den ? den + t0 * groups : nullptr, (T*)out + t0 * inner));
  }
  return nvs_check_launch("nvs_gated_group_norm");
}
