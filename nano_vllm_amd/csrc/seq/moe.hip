// Gated feed-forward activations and routed mixtures of experts.
//
// A routed layer runs as: router logits (a 32-bit library product) -> route kernel (softmax, choice scores, group limit,
// top-k, weights) -> plan kernel (pairs (token, choice) sorted by expert into row tiles, every expert's rows padded to a whole
// tile) -> grouped product gate|up with the activation in its epilogue -> grouped product down -> combine kernel (weighted sum
// of a token's choices, pass-through experts, the gated shared expert). Nothing comes back to the host in between, so the
// sequence can be captured in a hipGraph; the order in which pairs land inside an expert's rows is arbitrary but no sum depends
// on it (a row is computed on its own, and a token's choices are added in the order of its choices).
#include "seq_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

constexpr int MAX_EXPERTS = 1024;

__device__ __forceinline__ float glu_value(float g, float u, int kind, float limit, float alpha) {
  if (kind == 0) return g / (1.f + expf(-g)) * u;               // silu(g) * u
  if (kind == 2) return gelu_tanhf_(g);                         // ungated: the tanh form of GELU (u is not read)
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + 1.f);              // clamped: g sigmoid(alpha g) (u + 1)
}

// ungated products: mode 2 squares the positive part (the input rows are then gathered by token, as for a gated product)
__device__ __forceinline__ float plain_value(float v, int mode) {
  if (mode != 2) return v;
  v = fmaxf(v, 0.f);
  return v * v;
}

template <typename T>
__global__ void glu_act_kernel(const T* __restrict__ gu, int64_t stride, int ff, int kind, float limit, float alpha, int64_t n,
                               T* __restrict__ out) {
  const int64_t total = n * ff;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / ff;
    const int c = (int)(i - t * ff);
    stf(out + i, glu_value(ldf(gu + t * stride + c), kind == 2 ? 0.f : ldf(gu + t * stride + ff + c), kind, limit, alpha));
  }
}

// ---- routing without a router: a table row per token id names the token's experts, all with the same weight ----------
__global__ void moe_table_route_kernel(const int64_t* __restrict__ tokens, const int32_t* __restrict__ table, int64_t pairs, int top,
                                       float weight, int32_t* __restrict__ ids, float* __restrict__ wts) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= pairs) return;
  const int64_t t = i / top;
  ids[i] = table[tokens[t] * top + (i - t * top)];
  wts[i] = weight;
}

// ---- routing: one wavefront per token, a lane holds entries lane, lane + 64, ... of the token's scores ---------------
constexpr int ROUTE_PER_LANE = MAX_EXPERTS / 64;

__global__ void moe_route_kernel(const float* __restrict__ z, int64_t z_stride, const float* __restrict__ correction, int total,
                                 int top, int count, int keep, float scale, int score, int renorm, int32_t* __restrict__ ids,
                                 float* __restrict__ wts) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  const int per = total / count;
  float s[ROUTE_PER_LANE], c[ROUTE_PER_LANE];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < ROUTE_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    s[i] = e < total ? z[t * z_stride + e] : -INFINITY;
    mx = fmaxf(mx, s[i]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < ROUTE_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    if (score == 1) s[i] = e < total ? 1.f / (1.f + expf(-s[i])) : 0.f;      // sigmoid: every entry on its own
    else s[i] = e < total ? expf(s[i] - mx) : 0.f;
    sum += s[i];
  }
  sum = score == 1 ? 1.f : wave_sum(sum);
#pragma unroll
  for (int i = 0; i < ROUTE_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    s[i] = s[i] / sum;
    c[i] = e < total ? s[i] + (correction ? correction[e] : 0.f) : -INFINITY;      // the choice score; weights use s
  }
  if (count > 1) {
    // a group's score is its best choice score; entries outside the `keep` best groups cannot be chosen. Lane l holds the
    // score of group l (count <= 64) and ranks it: the number of groups that beat it, a lower index winning a tie.
    float mine = -INFINITY;
    for (int g = 0; g < count; ++g) {
      float v = -INFINITY;
#pragma unroll
      for (int i = 0; i < ROUTE_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        if (e < total && e / per == g) v = fmaxf(v, c[i]);
      }
      v = wave_max(v);
      if (lane == g) mine = v;
    }
    int better = 0;
    for (int g = 0; g < count; ++g) {
      const float v = __shfl(mine, g, 64);
      if (g != lane && (v > mine || (v == mine && g < lane))) ++better;
    }
    const int dropped = better >= keep;
    for (int g = 0; g < count; ++g) {
      if (__shfl(dropped, g, 64) == 0) continue;
#pragma unroll
      for (int i = 0; i < ROUTE_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        if (e < total && e / per == g) c[i] = -INFINITY;
      }
    }
  }
  float chosen_s = 0.f;                             // lane k: the score of choice k
  int chosen_e = 0;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
      const int e = lane + 64 * i;
      if (e < total && (c[i] > best)) best = c[i], at = e;      // (entries of a lane ascend: the first best stays)
    }
    const float wbest = wave_max(best);
    int cand = best == wbest ? at : 0x7fffffff;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const int other = __shfl_xor(cand, o, 64);
      cand = other < cand ? other : cand;
    }
    if (cand == 0x7fffffff) cand = 0;               // (fewer choosable entries than choices: cannot happen with valid sizes)
    float sv = 0.f;
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
      const int e = lane + 64 * i;
      if (e == cand) sv = s[i], c[i] = -INFINITY;
    }
    sv = wave_sum(sv);                              // one lane holds it
    if (lane == k) chosen_s = sv, chosen_e = cand;
  }
  const float denom = renorm ? wave_sum(lane < top ? chosen_s : 0.f) + 1e-20f : 1.f;
  if (lane < top) {
    ids[t * top + lane] = chosen_e;
    wts[t * top + lane] = chosen_s / denom * scale;
  }
}

// ---- plan: one workgroup sorts the pairs by expert --------------------------------------------------------------------
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int32_t* __restrict__ ids, int64_t pairs, int top, int experts, int tm,
                                                        int64_t cap, int32_t* __restrict__ tile_expert, int32_t* __restrict__ row_token,
                                                        int32_t* __restrict__ pair_row) {
  __shared__ int counts[MAX_EXPERTS];
  __shared__ int offs[MAX_EXPERTS + 1];
  const int tid = threadIdx.x, nt = blockDim.x;
  for (int e = tid; e < experts; e += nt) counts[e] = 0;
  for (int64_t r = tid; r < cap; r += nt) row_token[r] = -1;
  __syncthreads();
  for (int64_t i = tid; i < pairs; i += nt) {
    const int e = ids[i];
    if (e < experts) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int o = 0;
    for (int e = 0; e < experts; ++e) {
      offs[e] = o;
      o += (counts[e] + tm - 1) / tm * tm;
    }
    offs[experts] = o;
  }
  __syncthreads();
  for (int64_t tile = tid; tile < cap / tm; tile += nt) {
    const int64_t r = tile * tm;
    int e = -1;
    if (r < offs[experts]) {
      int lo = 0, hi = experts - 1;                 // the last expert whose offset is <= r and who has rows
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (offs[mid] <= r) lo = mid; else hi = mid - 1;
      }
      e = lo;
    }
    tile_expert[tile] = e;
  }
  for (int e = tid; e < experts; e += nt) counts[e] = offs[e];         // now the cursors
  __syncthreads();
  for (int64_t i = tid; i < pairs; i += nt) {
    const int e = ids[i];
    int r = -1;
    if (e < experts) {
      r = atomicAdd(&counts[e], 1);
      row_token[r] = (int32_t)(i / top);
    }
    pair_row[i] = r;
  }
}

// ---- grouped products --------------------------------------------------------------------------------------------------
// out[r, f] = sum_k X[src(r), k] * W[e(r)][f, k] for the rows r of a tile (all of one expert). GLU: W holds gate rows
// [0, nout) then up rows [nout, 2 nout) and the output is act(gate) * up; src(r) = row_token[r] (the token's input row),
// otherwise src(r) = r. Rows with row_token[r] < 0 are padding.

// plain form, any type and size: a thread owns one row and four features
template <typename T, bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const T* __restrict__ X, int64_t ldx, const T* __restrict__ W, int nout, int K,
                                                       const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ row_token,
                                                       int tm, T* __restrict__ out, int64_t ldo, int mode) {
  const int tiles_per = tm / 16;
  const int tile = blockIdx.x / tiles_per;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int64_t r = (int64_t)blockIdx.x * 16 + (threadIdx.x & 15);
  const int tok = row_token[r];
  if (tok < 0) return;
  const int64_t src = (GLU || mode == 2) ? tok : r;
  const T* xr = X + src * ldx;
  const T* We = W + (int64_t)e * (GLU ? 2 : 1) * nout * K;
  const int f0 = blockIdx.y * 64 + (threadIdx.x >> 4) * 4;
  float ag[4] = {0.f, 0.f, 0.f, 0.f}, au[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < K; ++k) {
    const float x = ldf(xr + k);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (f0 + i < nout) {
        ag[i] += x * ldf(We + (int64_t)(f0 + i) * K + k);
        if (GLU) au[i] += x * ldf(We + (int64_t)(nout + f0 + i) * K + k);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (f0 + i < nout) stf(out + r * ldo + f0 + i, GLU ? glu_value(ag[i], au[i], 0, 0.f, 0.f) : plain_value(ag[i], mode));
}

// matrix-core form (bf16, K % 8 == 0, 16-byte aligned rows). Computed transposed, C^T[features x rows] = W X^T with
// v_mfma_f32_16x16x32_bf16: the A operand is 16 weight rows x 32 of k, the B operand 16 input rows x 32 of k, both 16-byte
// loads straight from memory; a lane ends up with four consecutive features of one row (an 8-byte store). A workgroup of four
// wavefronts covers 16 MT rows x 128 features: every wavefront 32 features (FT = 2 blocks) for all the rows.
template <int MT, bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(const bf16_t* __restrict__ X, int64_t ldx, const bf16_t* __restrict__ W, int nout,
                                                            int K, const int32_t* __restrict__ tile_expert,
                                                            const int32_t* __restrict__ row_token, bf16_t* __restrict__ out, int64_t ldo, int mode) {
  constexpr int FT = 2, NG = GLU ? 2 : 1;
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 15, lk = (lane >> 4) * 8;
  const int64_t row0 = (int64_t)blockIdx.x * (16 * MT);
  const bf16_t* xp[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int64_t r = row0 + mt * 16 + li;
    const int tok = row_token[r];
    xok[mt] = tok >= 0;
    xp[mt] = X + (xok[mt] ? ((GLU || mode == 2) ? (int64_t)tok : r) : 0) * ldx + lk;
  }
  const bf16_t* We = W + (int64_t)e * NG * nout * K;
  const int fbase = blockIdx.y * (64 * FT) + wave * (16 * FT);
  const bf16_t* wp[FT];
  bool wok[FT];
#pragma unroll
  for (int ft = 0; ft < FT; ++ft) {
    const int f = fbase + ft * 16 + li;
    wok[ft] = f < nout;
    wp[ft] = We + (int64_t)(wok[ft] ? f : 0) * K + lk;
  }
  f32x4_t acc[NG][FT][MT];
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int ft = 0; ft < FT; ++ft)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[g][ft][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const bf16x8_t zero8 = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool kin = k0 + lk < K;
    bf16x8_t xb[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xb[mt] = (kin && xok[mt]) ? *(const bf16x8_t*)(xp[mt] + k0) : zero8;
#pragma unroll
    for (int ft = 0; ft < FT; ++ft) {
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const bf16x8_t wa = (kin && wok[ft]) ? *(const bf16x8_t*)(wp[ft] + (int64_t)g * nout * K + k0) : zero8;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[g][ft][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xb[mt], acc[g][ft][mt], 0, 0, 0);
      }
    }
  }
  // lane: row li of the tile block, features fbase + 16 ft + 4 (lane >> 4) + 0..3
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (!xok[mt]) continue;
    const int64_t r = row0 + mt * 16 + li;
#pragma unroll
    for (int ft = 0; ft < FT; ++ft) {
      const int f = fbase + ft * 16 + (lane >> 4) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (f + i < nout) {
          const float v = GLU ? glu_value(acc[0][ft][mt][i], acc[NG - 1][ft][mt][i], 0, 0.f, 0.f) : plain_value(acc[0][ft][mt][i], mode);
          out[r * ldo + f + i] = (bf16_t)v;
        }
      }
    }
  }
}

// LDS-tiled matrix-core form for steps with many rows per expert (tiles of 128 rows). A workgroup of four wavefronts computes
// 128 rows x 128 features (GLU: gate and up of the same 64 features; 128 weight rows either way) in steps of 64 along k: all
// threads load the step's operands with 16-byte loads — the NEXT step's loads are issued before the current step is computed —
// into LDS as [row][64 + 8]; a wavefront owns 64 rows x 64 weight rows (4 x 4 MFMA tiles) and reads its operands as 16-byte LDS
// reads: 16 reads for 32 MFMAs per step. The grid is one-dimensional and XCD-aware: workgroups are dealt to the eight XCDs
// round-robin, so workgroup id -> (id % 8) * per_xcd + id / 8 gives every XCD a CONTIGUOUS run of tiles, ordered feature tile
// major / row tile minor: consecutive tiles of an XCD share a weight tile (all row tiles of one expert), which its L2 then serves.
template <bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_tiled_kernel(const bf16_t* __restrict__ X, int64_t ldx, const bf16_t* __restrict__ W, int nout,
                                                             int K, const int32_t* __restrict__ tile_expert,
                                                             const int32_t* __restrict__ row_token, int tiles_m, int tiles_n,
                                                             bf16_t* __restrict__ out, int64_t ldo, int mode) {
  constexpr int BM = 128, BW = 128, BK = 64, LDK = BK + 8, NG = GLU ? 2 : 1, FB = 4 / NG, BN = BW / NG;   // BN features per tile
  __shared__ __attribute__((aligned(16))) bf16_t Xs[BM][LDK];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[BW][LDK];      // GLU: rows [0, 64) gate, [64, 128) up of the tile's features
  const int per_xcd = gridDim.x / 8;
  const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (logical >= tiles_m * tiles_n) return;
  const int rt = logical % tiles_m, ft = logical / tiles_m;
  const int e = tile_expert[rt];
  if (e < 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, lk = (lane >> 4) * 8;
  const int wm = wave & 1, wn = wave >> 1;
  const int64_t row0 = (int64_t)rt * BM;
  const bf16_t* We = W + (int64_t)e * NG * nout * K;
  // staging: unit u = tid + 256 i -> (row u >> 3, 8 elements of k at (u & 7) * 8); four units of each operand per thread
  const int sk = (tid & 7) * 8, sr = tid >> 3;
  const bf16_t* xsrc[4];
  const bf16_t* wsrc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = sr + 32 * i;
    const int tok = row_token[row0 + r];
    xsrc[i] = tok >= 0 ? X + ((GLU || mode == 2) ? (int64_t)tok : row0 + r) * ldx + sk : nullptr;
    const int g = r / BN, f = ft * BN + r % BN;
    wsrc[i] = f < nout ? We + ((int64_t)g * nout + f) * K + sk : nullptr;
  }
  const u32x4_t zero4 = u32x4_t{0u, 0u, 0u, 0u};
  u32x4_t xr[4], wr[4];
  auto fetch = [&](int k0) {
    const bool kin = k0 + sk < K;
#pragma unroll
    for (int i = 0; i < 4; ++i) xr[i] = (kin && xsrc[i]) ? *(const u32x4_t*)(xsrc[i] + k0) : zero4;
#pragma unroll
    for (int i = 0; i < 4; ++i) wr[i] = (kin && wsrc[i]) ? *(const u32x4_t*)(wsrc[i] + k0) : zero4;
  };
  // accumulators: weight-row block wb of this wavefront's 64 weight rows x row block rb. GLU: a wavefront's 64 weight rows are
  // 32 gate rows and the 32 up rows of the SAME features (wb 0, 1 gate; 2, 3 up), so the activation needs no exchange.
  f32x4_t acc[4][4];
#pragma unroll
  for (int wb = 0; wb < 4; ++wb)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) acc[wb][rb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  int wrow[4];                                      // LDS row of this lane's operand for weight-row block wb
#pragma unroll
  for (int wb = 0; wb < 4; ++wb) wrow[wb] = GLU ? (wb / FB) * BN + wn * 32 + (wb % FB) * 16 + li : wn * 64 + wb * 16 + li;
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();                                // the previous step's readers are done
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *(u32x4_t*)&Xs[sr + 32 * i][sk] = xr[i];
      *(u32x4_t*)&Ws[sr + 32 * i][sk] = wr[i];
    }
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 32) {
      bf16x8_t xb[4];
#pragma unroll
      for (int rb = 0; rb < 4; ++rb) xb[rb] = *(const bf16x8_t*)&Xs[wm * 64 + rb * 16 + li][kk + lk];
#pragma unroll
      for (int wb = 0; wb < 4; ++wb) {
        const bf16x8_t wa = *(const bf16x8_t*)&Ws[wrow[wb]][kk + lk];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) acc[wb][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xb[rb], acc[wb][rb], 0, 0, 0);
      }
    }
  }
  // lane: row li of row block rb; features 16 fb + 4 (lane >> 4) + 0..3 of its wavefront's 64 (GLU: 32)
#pragma unroll
  for (int rb = 0; rb < 4; ++rb) {
    const int64_t r = row0 + wm * 64 + rb * 16 + li;
    if (row_token[r] < 0) continue;
#pragma unroll
    for (int fb = 0; fb < FB; ++fb) {
      const int f = ft * BN + wn * (16 * FB) + fb * 16 + (lane >> 4) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (f + i < nout) {
          const float v = GLU ? glu_value(acc[fb][rb][i], acc[GLU ? fb + FB : fb][rb][i], 0, 0.f, 0.f) : plain_value(acc[fb][rb][i], mode);
          out[r * ldo + f + i] = (bf16_t)v;
        }
      }
    }
  }
}

// ---- combine: one workgroup per token ------------------------------------------------------------------------------------
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ rows, int64_t ldr, const int32_t* __restrict__ pair_row,
                                   const float* __restrict__ wts, int top, const T* __restrict__ h, int64_t ldh,
                                   const T* __restrict__ shared, const float* __restrict__ shared_gate, int64_t gate_stride, int width,
                                   T* __restrict__ out) {
  const int64_t t = blockIdx.x;
  float sg = 0.f;
  if (shared) sg = shared_gate ? 1.f / (1.f + expf(-shared_gate[t * gate_stride])) : 1.f;      // no gate: the shared expert is added as it is
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int r = pair_row[t * top + k];
      const float v = r >= 0 ? ldf(rows + (int64_t)r * ldr + c) : ldf(h + t * ldh + c);      // no row: a pass-through expert
      acc += wts[t * top + k] * v;
    }
    if (shared) acc += sg * ldf(shared + t * width + c);
    stf(out + t * width + c, acc);
  }
}

}  // namespace

static int g_moe_plain = 0;
extern "C" void nvs_moe_force_plain(int on) { g_moe_plain = on; }

extern "C" int nvs_glu_act(const void* gu, int64_t stride, int dtype, int ff, int kind, float limit, float alpha, int64_t n, void* out,
                           void* stream) {
  NVS_REQUIRE(gu && out && ff > 0 && stride >= (kind == 2 ? 1 : 2) * (int64_t)ff && kind >= 0 && kind <= 2 && n >= 0, "nvs_glu_act: ff %d stride %lld kind %d",
              ff, (long long)stride, kind);
  if (n == 0) return NVS_OK;
  int64_t blocks = (n * ff + 255) / 256;
  if (blocks > 65535 * 16) blocks = 65535 * 16;
  NVS_DISPATCH(dtype, glu_act_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>((const T*)gu, stride, ff, kind, limit,
                                                                                                    alpha, n, (T*)out));
  return nvs_check_launch("nvs_glu_act");
}

extern "C" int nvs_moe_route(const float* z, int64_t z_stride, const float* correction, int64_t n, int total, int top, int count, int keep,
                             float scale, int score, int renorm, int32_t* ids, float* wts, void* stream) {
  NVS_REQUIRE(z && ids && wts && n >= 0 && (score == 0 || score == 1), "nvs_moe_route: bad argument");
  NVS_REQUIRE(total > 0 && total <= MAX_EXPERTS && z_stride >= total && top > 0 && top <= 64 && count > 0 && count <= 64 && total % count == 0 &&
                  keep > 0 && keep <= count && (int64_t)keep * (total / count) >= top,
              "nvs_moe_route: %d entries, %d choices, %d of %d groups", total, top, keep, count);
  if (n == 0) return NVS_OK;
  moe_route_kernel<<<dim3((unsigned)n), dim3(64), 0, (hipStream_t)stream>>>(z, z_stride, correction, total, top, count, keep, scale, score, renorm, ids, wts);
  return nvs_check_launch("nvs_moe_route");
}

extern "C" int nvs_moe_table_route(const int64_t* tokens, const int32_t* table, int64_t n, int top, float weight, int32_t* ids, float* wts,
                                   void* stream) {
  NVS_REQUIRE(tokens && table && ids && wts && n >= 0 && top > 0 && top <= 64, "nvs_moe_table_route: bad argument (%d choices)", top);
  if (n == 0) return NVS_OK;
  const int64_t pairs = n * top;
  moe_table_route_kernel<<<dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(tokens, table, pairs, top, weight, ids, wts);
  return nvs_check_launch("nvs_moe_table_route");
}

extern "C" int64_t nvs_moe_rows(int64_t pairs, int experts, int tm) { return (pairs + (int64_t)experts * (tm - 1) + tm - 1) / tm * tm; }

extern "C" int nvs_moe_plan(const int32_t* ids, int64_t n, int top, int experts, int tm, int32_t* tile_expert, int32_t* row_token,
                            int32_t* pair_row, void* stream) {
  NVS_REQUIRE(ids && tile_expert && row_token && pair_row && n >= 0 && top > 0, "nvs_moe_plan: null argument");
  NVS_REQUIRE(experts > 0 && experts <= MAX_EXPERTS && (tm == 16 || tm == 64 || tm == 128), "nvs_moe_plan: %d experts, tiles of %d rows", experts, tm);
  if (n == 0) return NVS_OK;
  const int64_t cap = nvs_moe_rows(n * top, experts, tm);
  NVS_REQUIRE(cap < (1ll << 31), "nvs_moe_plan: step too large");
  moe_plan_kernel<<<dim3(1), dim3(1024), 0, (hipStream_t)stream>>>(ids, n * top, top, experts, tm, cap, tile_expert, row_token, pair_row);
  return nvs_check_launch("nvs_moe_plan");
}

extern "C" int nvs_moe_gemm(const void* X, int64_t ldx, const void* W, int dtype, int mode, int nout, int K, const int32_t* tile_expert,
                            const int32_t* row_token, int64_t cap, int tm, void* out, int64_t ldo, void* stream) {
  NVS_REQUIRE(X && W && tile_expert && row_token && out && mode >= 0 && mode <= 2, "nvs_moe_gemm: bad argument");
  const int glu = mode == 1;
  NVS_REQUIRE(nout > 0 && K > 0 && ldx >= K && ldo >= nout && (tm == 16 || tm == 64 || tm == 128) && cap >= 0 && cap % tm == 0,
              "nvs_moe_gemm: %d x %d, %lld rows in tiles of %d", nout, K, (long long)cap, tm);
  if (cap == 0) return NVS_OK;
  hipStream_t st = (hipStream_t)stream;
  const bool matrix_cores = dtype == NVS_BF16 && K % 8 == 0 && ldx % 8 == 0 && !g_moe_plain;
  if (matrix_cores && tm == 128) {
    const int bn = glu ? 64 : 128;                  // features per tile
    const int tiles_m = (int)(cap / 128), tiles_n = (nout + bn - 1) / bn;
    const int64_t blocks = ((int64_t)tiles_m * tiles_n + 7) / 8 * 8;
    NVS_REQUIRE(blocks < (1ll << 31), "nvs_moe_gemm: step too large");
    if (glu)
      moe_gemm_tiled_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((const bf16_t*)X, ldx, (const bf16_t*)W, nout, K, tile_expert,
                                                                                row_token, tiles_m, tiles_n, (bf16_t*)out, ldo, mode);
    else
      moe_gemm_tiled_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((const bf16_t*)X, ldx, (const bf16_t*)W, nout, K, tile_expert,
                                                                                 row_token, tiles_m, tiles_n, (bf16_t*)out, ldo, mode);
    return nvs_check_launch("nvs_moe_gemm (matrix cores, LDS tiles)");
  }
  if (matrix_cores) {
    const dim3 grid((unsigned)(cap / tm), (unsigned)((nout + 127) / 128));
#define NVS_MOE_CASE(MT, GLU)                                                                                                        \
  moe_gemm_mfma_kernel<MT, GLU><<<grid, dim3(256), 0, st>>>((const bf16_t*)X, ldx, (const bf16_t*)W, nout, K, tile_expert, row_token,  \
                                                            (bf16_t*)out, ldo, mode)
    if (tm == 64) {
      if (glu) NVS_MOE_CASE(4, true); else NVS_MOE_CASE(4, false);
    } else {
      if (glu) NVS_MOE_CASE(1, true); else NVS_MOE_CASE(1, false);
    }
#undef NVS_MOE_CASE
    return nvs_check_launch("nvs_moe_gemm (matrix cores)");
  }
  const dim3 grid((unsigned)(cap / 16), (unsigned)((nout + 63) / 64));
  if (glu) {
    NVS_DISPATCH(dtype, moe_gemm_kernel<T, true><<<grid, dim3(256), 0, st>>>((const T*)X, ldx, (const T*)W, nout, K, tile_expert, row_token, tm,
                                                                            (T*)out, ldo, mode));
  } else {
    NVS_DISPATCH(dtype, moe_gemm_kernel<T, false><<<grid, dim3(256), 0, st>>>((const T*)X, ldx, (const T*)W, nout, K, tile_expert, row_token,
                                                                             tm, (T*)out, ldo, mode));
  }
  return nvs_check_launch("nvs_moe_gemm");
}

extern "C" int nvs_moe_combine(const void* rows, int64_t ldr, const int32_t* pair_row, const float* wts, int top, const void* h, int64_t ldh,
                               const void* shared, const float* shared_gate, int64_t gate_stride, int dtype, int64_t n, int width, void* out,
                               void* stream) {
  NVS_REQUIRE(rows && pair_row && wts && h && out && top > 0 && width > 0 && n >= 0,
              "nvs_moe_combine: bad argument");
  if (n == 0) return NVS_OK;
  const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
  NVS_DISPATCH(dtype, moe_combine_kernel<T><<<dim3((unsigned)n), dim3(threads), 0, (hipStream_t)stream>>>(
                          (const T*)rows, ldr, pair_row, wts, top, (const T*)h, ldh, (const T*)shared, shared_gate, gate_stride, width,
                          (T*)out));
  return nvs_check_launch("nvs_moe_combine");
}
