// A feed-forward of many small gated experts of which every token uses a few:
//   router_choice   s = softmax(z) over all router outputs; the `top` largest of s + correction
//                   are chosen (the lower index on a tie); their weights are s itself.
//   silu_mul        act = silu(gate) * up for rows [gate | up]   (a dense gated feed-forward)
//   route_and_gate  both of these in one launch, for a step of few tokens whose router, gate and up
//                   came out of one product as float rows
//   expert_rows_up / expert_rows_down
//                   a token's chosen experts read straight from the stacked expert weights, a
//                   wave four features at once: act[t, j, :] = w_tj silu(Wg_e x_t) * (Wu_e x_t), then
//                   y[t, :] += sum_j Wd_e act[t, j, :] + sum_(j: e is an identity expert) w_tj x_t.
//                   Only the chosen experts' weights are read: the kernels for few tokens.
//   expert_tiles    the same for many tokens: the picks are sorted by expert on the device
//                   (expert_sort: counts, offsets, tiles of up to 64 picks of one expert), and
//                   every tile is a small matrix product on the matrix cores with the rows
//                   gathered through the sorted list: [gate | up] with the activation and the
//                   pick's weight in the epilogue, then down into a row of its own for every
//                   pick; expert_combine adds a token's picks in their order, and the identity
//                   experts' share.  The grid is as large as the tiles could be at most; blocks
//                   beyond the tiles that there are leave at once, so nothing comes to the host.
// The router's softmax, the choice and the weights are 32-bit; products accumulate in 32-bit.
#include "common.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

// A wave a token, up to ROUTER_PER_LANE outputs a lane.  The k-th pick is the largest choice score
// not picked yet, the lowest index on a tie.
#define ROUTER_PER_LANE 8
// `renorm`: the picks' weights are divided by their sum (+ 1e-20); `mult`: and multiplied by this.
__device__ __forceinline__ void route_token(const float* __restrict__ zr, const float* __restrict__ correction, int n_out,
                                            int top, int* __restrict__ idx, float* __restrict__ weight, int lane,
                                            int renorm = 0, float mult = 1.f) {
  float v[ROUTER_PER_LANE], c[ROUTER_PER_LANE];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < ROUTER_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < n_out ? zr[e] : -INFINITY;
    m = fmaxf(m, v[i]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < ROUTER_PER_LANE; ++i) {
    v[i] = lane + 64 * i < n_out ? expf(v[i] - m) : 0.f;
    sum += v[i];
  }
  const float inv = 1.0f / wave_sum(sum);
#pragma unroll
  for (int i = 0; i < ROUTER_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    v[i] *= inv;
    c[i] = e < n_out ? (correction ? v[i] + correction[e] : v[i]) : -INFINITY;
  }
  float mine[ROUTER_PER_LANE];  // pick j's weight, kept by lane j % 64 until the picks' sum is known
#pragma unroll
  for (int i = 0; i < ROUTER_PER_LANE; ++i) mine[i] = 0.f;
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
#pragma unroll
    for (int i = 0; i < ROUTER_PER_LANE; ++i) best = fmaxf(best, c[i]);
    best = wave_max(best);
    float first = -1e9f;  // minus the lowest index that holds the best score (indices are exact in a float)
#pragma unroll
    for (int i = ROUTER_PER_LANE - 1; i >= 0; --i)
      if (c[i] == best) first = -(float)(lane + 64 * i);
    const int e = (int)(-wave_max(first));
    float w = 0.f;
#pragma unroll
    for (int i = 0; i < ROUTER_PER_LANE; ++i)
      if (lane + 64 * i == e) {
        idx[j] = e, w = v[i];
        c[i] = -INFINITY;  // picked
      }
    w = wave_sum(w);  // (one lane holds it)
    total += w;
#pragma unroll
    for (int i = 0; i < ROUTER_PER_LANE; ++i)
      if (lane == (j & 63) && i == (j >> 6)) mine[i] = w;
  }
  const float factor = renorm ? mult / (total + 1e-20f) : mult;
#pragma unroll
  for (int i = 0; i < ROUTER_PER_LANE; ++i)
    if (lane + 64 * i < top) weight[lane + 64 * i] = mine[i] * factor;
}

__global__ __launch_bounds__(256) void router_choice_kernel(const float* __restrict__ z, int ldz,
                                                            const float* __restrict__ correction, int n_tokens,
                                                            int n_out, int top, int* __restrict__ idx,
                                                            float* __restrict__ weight, int renorm, float mult) {
  const int lane = threadIdx.x & 63, t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= n_tokens) return;  // whole waves leave; no barrier follows
  route_token(z + (size_t)t * ldz, correction, n_out, top, idx + (size_t)t * top, weight + (size_t)t * top, lane, renorm, mult);
}

// For a step of few tokens, where one product gave [router | gate | up] as float rows: a block a
// token, its first wave chooses the experts, all of it makes act = silu(gate) * up.
template <typename T>
__global__ __launch_bounds__(256) void route_and_gate_kernel(const float* __restrict__ zu, int ld,
                                                             const float* __restrict__ correction, int n_out, int top,
                                                             int F, int* __restrict__ idx, float* __restrict__ weight,
                                                             T* __restrict__ act, int ldo, int renorm, float mult) {
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  const float* row = zu + (size_t)t * ld;
  if (threadIdx.x < 64)
    route_token(row, correction, n_out, top, idx + (size_t)t * top, weight + (size_t)t * top, lane, renorm, mult);
  for (int f = threadIdx.x; f < F; f += 256) act[(size_t)t * ldo + f] = from_f32<T>(silu_f(row[n_out + f]) * row[n_out + F + f]);
}

// GELU: the gate passes the tanh form of gelu instead of silu
template <typename T, bool GELU>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ gu, int ld, T* __restrict__ out, int ldo,
                                                       int n_rows, int F) {
  const int f = blockIdx.y * 256 + threadIdx.x, r = blockIdx.x;
  if (f >= F) return;
  const T* row = gu + (size_t)r * ld;
  const float z = to_f32(row[f]);
  out[(size_t)r * ldo + f] = from_f32<T>((GELU ? gelu_tanh(z) : silu_f(z)) * to_f32(row[F + f]));
}

// ROWS dot products of one vector b with ROWS rows a[r] over a lane's share of K, all loads of a step on
// their way at once: 16 bytes a lane and load where K and the rows allow (VEC), a value a lane otherwise.
template <typename T, bool VEC, int ROWS>
__device__ __forceinline__ void lane_dots(const T* const* __restrict__ a, const T* __restrict__ b, int K, int lane, float* s) {
#pragma unroll
  for (int r = 0; r < ROWS; ++r) s[r] = 0.f;
  if (VEC) {
    constexpr int W = 16 / sizeof(T);
    for (int k = lane * W; k < K; k += 64 * W) {
      u32x4_t av[ROWS];
      const u32x4_t bv = *(const u32x4_t*)(b + k);
#pragma unroll
      for (int r = 0; r < ROWS; ++r) av[r] = *(const u32x4_t*)(a[r] + k);
      const T* bp = (const T*)&bv;
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const T* ap = (const T*)&av[r];
#pragma unroll
        for (int i = 0; i < W; ++i) s[r] += to_f32(ap[i]) * to_f32(bp[i]);
      }
    }
  } else {
    for (int k = lane; k < K; k += 64) {
      const float bv = to_f32(b[k]);
#pragma unroll
      for (int r = 0; r < ROWS; ++r) s[r] += to_f32(a[r][k]) * bv;
    }
  }
}

// Block (token x pick, 16 features): a wave four features at once (eight rows of weights in
// flight), lanes along the width.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void expert_rows_up_kernel(const T* __restrict__ x, int ldx,
                                                             const T* __restrict__ w_gate, const T* __restrict__ w_up,
                                                             const int* __restrict__ idx,
                                                             const float* __restrict__ weight, int n_experts, int top,
                                                             int F, int width, T* __restrict__ act) {
  const int item = blockIdx.x, t = item / top;
  const int e = idx[item];
  if (e >= n_experts) return;  // an identity expert: nothing to compute
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int f0 = blockIdx.y * 16 + wave * 4;
  if (f0 >= F) return;  // (no barrier in this kernel)
  const T* rows[8];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const size_t f = (size_t)e * F + min(f0 + r, F - 1);
    rows[r] = w_gate + f * width, rows[4 + r] = w_up + f * width;
  }
  float s[8];
  lane_dots<T, VEC, 8>(rows, x + (size_t)t * ldx, width, lane, s);
#pragma unroll
  for (int r = 0; r < 8; ++r) s[r] = wave_sum(s[r]);
  const float wt = weight[item];
  if (lane < 4 && f0 + lane < F) {
    float g = s[0], u = s[4];
#pragma unroll
    for (int r = 1; r < 4; ++r)
      if (lane == r) g = s[r], u = s[4 + r];
    act[(size_t)item * F + f0 + lane] = from_f32<T>(wt * silu_f(g) * u);
  }
}

// Block (token, 16 columns): a wave four output columns at once, lanes along the features.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void expert_rows_down_kernel(const T* __restrict__ act, const T* __restrict__ w_down,
                                                               const int* __restrict__ idx,
                                                               const float* __restrict__ weight,
                                                               const T* __restrict__ x, int ldx, int n_experts, int top,
                                                               int F, int width, float* __restrict__ y, int ldy,
                                                               int accumulate) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = blockIdx.y * 16 + wave * 4;
  if (n0 >= width) return;
  float tot[4] = {0.f, 0.f, 0.f, 0.f}, same = 0.f;
  for (int j = 0; j < top; ++j) {
    const int e = idx[(size_t)t * top + j];
    if (e >= n_experts) {
      same += weight[(size_t)t * top + j];
      continue;
    }
    const T* rows[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) rows[r] = w_down + ((size_t)e * width + min(n0 + r, width - 1)) * F;
    float s[4];
    lane_dots<T, VEC, 4>(rows, act + ((size_t)t * top + j) * F, F, lane, s);
#pragma unroll
    for (int r = 0; r < 4; ++r) tot[r] += s[r];
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) tot[r] = wave_sum(tot[r]);
  if (lane < 4 && n0 + lane < width) {
    float v = tot[0];
#pragma unroll
    for (int r = 1; r < 4; ++r)
      if (lane == r) v = tot[r];
    v += same * to_f32(x[(size_t)t * ldx + n0 + lane]);
    float* o = y + (size_t)t * ldy + n0 + lane;
    *o = accumulate ? *o + v : v;
  }
}

// ---------------------------------------------------------------------------
// many tokens: picks sorted by expert, a tile of picks a block

#define TILE_PICKS 64

// One block.  tiles: (expert, first place in `order`, picks) each.
__global__ __launch_bounds__(1024) void expert_sort_kernel(const int* __restrict__ idx, int n_items, int n_experts,
                                                           int* __restrict__ order, int* __restrict__ tiles,
                                                           int* __restrict__ n_tiles) {
  extern __shared__ int lds_i[];
  int* counts = lds_i;
  int* cursor = lds_i + n_experts;
  for (int e = threadIdx.x; e < n_experts; e += 1024) counts[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_items; i += 1024) {
    const int e = idx[i];
    if (e < n_experts) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < n_experts; ++e) {
      cursor[e] = at;
      for (int r0 = 0; r0 < counts[e]; r0 += TILE_PICKS) {
        tiles[3 * nt] = e, tiles[3 * nt + 1] = at + r0, tiles[3 * nt + 2] = min(TILE_PICKS, counts[e] - r0);
        ++nt;
      }
      at += counts[e];
    }
    *n_tiles = nt;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n_items; i += 1024) {
    const int e = idx[i];
    if (e < n_experts) order[atomicAdd(&cursor[e], 1)] = i;  // (any order within an expert: a pick's row is computed by itself)
  }
}

// A lane's share of a 16 x 16 product's operands: row (or column) lane % 16, KL values of k from
// KL * (lane / 16) on; the sums land as rows 4 (lane / 16) + i, column lane % 16.
template <typename T>
struct Frag;
template <>
struct Frag<bf16> {
  typedef bf16x8_t V;
  static constexpr int KL = 8;
  // (a lane beyond K brings zeros: the matrix instruction takes every lane's registers, whatever
  // the lanes' state, so the product itself must not stand under a condition)
  static __device__ __forceinline__ V load(const bf16* p, bool inside) {
    u32x4_t bits = {0u, 0u, 0u, 0u};
    if (inside) bits = *(const u32x4_t*)p;
    return __builtin_bit_cast(bf16x8_t, bits);
  }
  static __device__ __forceinline__ f32x4_t mma(V a, V b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Frag<float> {
  typedef f32x4_t V;
  static constexpr int KL = 4;
  static __device__ __forceinline__ V load(const float* p, bool inside) {
    f32x4_t v = {0.f, 0.f, 0.f, 0.f};
    if (inside) v = *(const f32x4_t*)p;
    return v;
  }
  static __device__ __forceinline__ f32x4_t mma(V a, V b, f32x4_t c) {
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, c, 0, 0, 0);
  }
};

// Block (tile, 64 CF features): a wave all of the tile's picks (four groups of 16) x 16 CF features
// of gate and of up, operands straight from memory; a weight fragment meets up to four fragments
// of rows.  CF = 4 where the tiles alone fill the GPU, 1 where they are few (a decode step of some
// dozen tokens), so that the blocks are four times as many.  act[pick, f] = weight * silu(gate) * up.
template <typename T, int CF>
__global__ __launch_bounds__(256) void expert_tiles_up_kernel(const T* __restrict__ x, int ldx, const T* __restrict__ w_gate,
                                                              const T* __restrict__ w_up, const int* __restrict__ order,
                                                              const int* __restrict__ tiles, const int* __restrict__ n_tiles,
                                                              const float* __restrict__ weight, int top, int F, int width,
                                                              T* __restrict__ act) {
  typedef Frag<T> Fr;
  if ((int)blockIdx.x >= *n_tiles) return;
  const int e = tiles[3 * blockIdx.x], first = tiles[3 * blockIdx.x + 1], count = tiles[3 * blockIdx.x + 2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, r = lane & 15;
  const int f0 = (blockIdx.y * 4 + wave) * 16 * CF;
  if (f0 >= F) return;  // (no barrier in this kernel)
  const int groups = (count + 15) / 16;
  const T* xrow[4];
#pragma unroll
  for (int rg = 0; rg < 4; ++rg) xrow[rg] = x + (size_t)(order[first + min(16 * rg + r, count - 1)] / top) * ldx;
  const T* grow[CF];
  const T* urow[CF];
#pragma unroll
  for (int c = 0; c < CF; ++c) {
    const size_t f = (size_t)e * F + min(f0 + 16 * c + r, F - 1);
    grow[c] = w_gate + f * width, urow[c] = w_up + f * width;
  }
  f32x4_t ag[4][CF], au[4][CF];
#pragma unroll
  for (int rg = 0; rg < 4; ++rg)
#pragma unroll
    for (int c = 0; c < CF; ++c) ag[rg][c] = au[rg][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // two sets of operands by turns: the next step's loads are on their way during this step's products
  // (the width is a multiple of KL: a lane's values are all inside or all outside)
  typename Fr::V a[2][4], bg[2][CF], bu[2][CF];
  const int step = 4 * Fr::KL;
#define LOAD_SET(S, K0)                                                                                 \
  do {                                                                                                  \
    const int k_ = (K0) + Fr::KL * g;                                                                   \
    const bool in_ = k_ < width;                                                                        \
    _Pragma("unroll") for (int rg = 0; rg < 4; ++rg) a[S][rg] = Fr::load(xrow[rg] + k_, in_);           \
    _Pragma("unroll") for (int c = 0; c < CF; ++c) bg[S][c] = Fr::load(grow[c] + k_, in_), bu[S][c] = Fr::load(urow[c] + k_, in_); \
  } while (0)
#define MMA_SET(S)                                                                                      \
  do {                                                                                                  \
    _Pragma("unroll") for (int rg = 0; rg < 4; ++rg) {                                                  \
      if (rg < groups) { /* (the same for every lane of the block) */                                   \
        _Pragma("unroll") for (int c = 0; c < CF; ++c) {                                                 \
          ag[rg][c] = Fr::mma(a[S][rg], bg[S][c], ag[rg][c]);                                           \
          au[rg][c] = Fr::mma(a[S][rg], bu[S][c], au[rg][c]);                                           \
        }                                                                                               \
      }                                                                                                 \
    }                                                                                                   \
  } while (0)
  LOAD_SET(0, 0);
  for (int k0 = 0; k0 < width; k0 += 2 * step) {
    LOAD_SET(1, k0 + step);  // (beyond the width: zeros, and nothing is read)
    MMA_SET(0);
    LOAD_SET(0, k0 + 2 * step);
    MMA_SET(1);
  }
#undef LOAD_SET
#undef MMA_SET
#pragma unroll
  for (int rg = 0; rg < 4; ++rg)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ri = 16 * rg + 4 * g + i;
      if (ri >= count) continue;
      const int it = order[first + ri];
      const float wt = weight[it];
#pragma unroll
      for (int c = 0; c < CF; ++c) {
        const int f = f0 + 16 * c + r;
        if (f < F) act[(size_t)it * F + f] = from_f32<T>(wt * silu_f(ag[rg][c][i]) * au[rg][c][i]);
      }
    }
}

// Block (tile, 64 CF columns): out[pick, n] = sum_f act[pick, f] w_down[e, n, f], laid out as above.
template <typename T, int CF>
__global__ __launch_bounds__(256) void expert_tiles_down_kernel(const T* __restrict__ act, const T* __restrict__ w_down,
                                                                const int* __restrict__ order, const int* __restrict__ tiles,
                                                                const int* __restrict__ n_tiles, int F, int width,
                                                                float* __restrict__ out) {
  typedef Frag<T> Fr;
  if ((int)blockIdx.x >= *n_tiles) return;
  const int e = tiles[3 * blockIdx.x], first = tiles[3 * blockIdx.x + 1], count = tiles[3 * blockIdx.x + 2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, r = lane & 15;
  const int n0 = (blockIdx.y * 4 + wave) * 16 * CF;
  if (n0 >= width) return;
  const int groups = (count + 15) / 16;
  const T* arow[4];
#pragma unroll
  for (int rg = 0; rg < 4; ++rg) arow[rg] = act + (size_t)order[first + min(16 * rg + r, count - 1)] * F;
  const T* drow[CF];
#pragma unroll
  for (int c = 0; c < CF; ++c) drow[c] = w_down + ((size_t)e * width + min(n0 + 16 * c + r, width - 1)) * F;
  f32x4_t acc[4][CF];
#pragma unroll
  for (int rg = 0; rg < 4; ++rg)
#pragma unroll
    for (int c = 0; c < CF; ++c) acc[rg][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  typename Fr::V a[2][4], b[2][CF];
  const int step = 4 * Fr::KL;
#define LOAD_SET(S, K0)                                                                        \
  do {                                                                                         \
    const int k_ = (K0) + Fr::KL * g;                                                          \
    const bool in_ = k_ < F;                                                                   \
    _Pragma("unroll") for (int rg = 0; rg < 4; ++rg) a[S][rg] = Fr::load(arow[rg] + k_, in_);  \
    _Pragma("unroll") for (int c = 0; c < CF; ++c) b[S][c] = Fr::load(drow[c] + k_, in_);       \
  } while (0)
#define MMA_SET(S)                                                                             \
  do {                                                                                         \
    _Pragma("unroll") for (int rg = 0; rg < 4; ++rg) {                                         \
      if (rg < groups) {                                                                       \
        _Pragma("unroll") for (int c = 0; c < CF; ++c) acc[rg][c] = Fr::mma(a[S][rg], b[S][c], acc[rg][c]); \
      }                                                                                        \
    }                                                                                          \
  } while (0)
  LOAD_SET(0, 0);
  for (int k0 = 0; k0 < F; k0 += 2 * step) {
    LOAD_SET(1, k0 + step);
    MMA_SET(0);
    LOAD_SET(0, k0 + 2 * step);
    MMA_SET(1);
  }
#undef LOAD_SET
#undef MMA_SET
#pragma unroll
  for (int rg = 0; rg < 4; ++rg)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ri = 16 * rg + 4 * g + i;
      if (ri >= count) continue;
      const size_t it = order[first + ri];
#pragma unroll
      for (int c = 0; c < CF; ++c) {
        const int n = n0 + 16 * c + r;
        if (n < width) out[it * width + n] = acc[rg][c][i];
      }
    }
}

// Thread (token, column): a token's picks in their order, identity experts give weight * x.
template <typename T>
__global__ __launch_bounds__(256) void expert_combine_kernel(const float* __restrict__ out, const int* __restrict__ idx,
                                                             const float* __restrict__ weight, const T* __restrict__ x, int ldx,
                                                             int n_experts, int top, int width, float* __restrict__ y, int ldy,
                                                             int accumulate) {
  const int n = blockIdx.y * 256 + threadIdx.x, t = blockIdx.x;
  if (n >= width) return;
  float s = 0.f, same = 0.f;
  for (int j = 0; j < top; ++j) {
    const size_t it = (size_t)t * top + j;
    if (idx[it] >= n_experts)
      same += weight[it];
    else
      s += out[it * width + n];
  }
  const float v = s + same * to_f32(x[(size_t)t * ldx + n]);
  float* o = y + (size_t)t * ldy + n;
  *o = accumulate ? *o + v : v;
}

DEFINE_LAST_ERROR(mlxlm_last_error)

static int router_choice_launch(const float* z, int ldz, const float* correction, int n_tokens, int n_out, int top,
                                int* idx, float* weight, int renorm, float mult, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (!z || !idx || !weight) FAIL("router_choice: null pointer");
  if (n_out <= 0 || top <= 0 || top > n_out || ldz < n_out) FAIL("router_choice: %d of %d outputs, rows of %d", top, n_out, ldz);
  if (n_out > 64 * ROUTER_PER_LANE) FAIL("router_choice: %d outputs, at most %d", n_out, 64 * ROUTER_PER_LANE);
  hipLaunchKernelGGL(router_choice_kernel, dim3((n_tokens + 3) / 4), dim3(256), 0, stream, z, ldz, correction,
                     n_tokens, n_out, top, idx, weight, renorm, mult);
  CHECK_LAUNCH("router_choice");
  return 0;
}

extern "C" int router_choice(const float* z, int ldz, const float* correction, int n_tokens, int n_out, int top,
                             int* idx, float* weight, hipStream_t stream) {
  return router_choice_launch(z, ldz, correction, n_tokens, n_out, top, idx, weight, 0, 1.f, stream);
}

// router_choice_scaled: the picks' weights divided by their sum (+ 1e-20) where `renorm`, then times `mult`.
extern "C" int router_choice_scaled(const float* z, int ldz, const float* correction, int n_tokens, int n_out, int top,
                                    int* idx, float* weight, int renorm, float mult, hipStream_t stream) {
  return router_choice_launch(z, ldz, correction, n_tokens, n_out, top, idx, weight, renorm, mult, stream);
}

static int route_and_gate_launch(const float* zu, int ld, const float* correction, int n_tokens, int n_out, int top, int F,
                                 int* idx, float* weight, void* act, int ldo, int dtype, int renorm, float mult,
                                 hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (!zu || !idx || !weight || !act) FAIL("route_and_gate: null pointer");
  if (n_out <= 0 || top <= 0 || top > n_out || F <= 0 || ld < n_out + 2 * F || ldo < F)
    FAIL("route_and_gate: %d of %d outputs and 2 x %d columns in rows of %d", top, n_out, F, ld);
  if (n_out > 64 * ROUTER_PER_LANE) FAIL("route_and_gate: %d outputs, at most %d", n_out, 64 * ROUTER_PER_LANE);
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("route_and_gate: unknown dtype code %d", dtype);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(route_and_gate_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, zu, ld, correction, n_out, top, F,
                       idx, weight, (float*)act, ldo, renorm, mult);
  else
    hipLaunchKernelGGL(route_and_gate_kernel<bf16>, dim3(n_tokens), dim3(256), 0, stream, zu, ld, correction, n_out, top, F,
                       idx, weight, (bf16*)act, ldo, renorm, mult);
  CHECK_LAUNCH("route_and_gate");
  return 0;
}

extern "C" int route_and_gate(const float* zu, int ld, const float* correction, int n_tokens, int n_out, int top, int F,
                              int* idx, float* weight, void* act, int ldo, int dtype, hipStream_t stream) {
  return route_and_gate_launch(zu, ld, correction, n_tokens, n_out, top, F, idx, weight, act, ldo, dtype, 0, 1.f, stream);
}

extern "C" int route_and_gate_scaled(const float* zu, int ld, const float* correction, int n_tokens, int n_out, int top,
                                     int F, int* idx, float* weight, void* act, int ldo, int dtype, int renorm, float mult,
                                     hipStream_t stream) {
  return route_and_gate_launch(zu, ld, correction, n_tokens, n_out, top, F, idx, weight, act, ldo, dtype, renorm, mult, stream);
}

// act_mul: out = act(gate) * up for rows [gate | up]; `activation` 0: silu, 1: the tanh form of gelu.
static int act_mul_launch(const void* gu, int ld, void* out, int ldo, int n_rows, int F, int dtype, int activation,
                          hipStream_t stream) {
  if (n_rows <= 0 || F <= 0) return 0;
  if (activation != 0 && activation != 1) FAIL("act_mul: unknown activation code %d", activation);
  if (!gu || !out) FAIL("silu_mul: null pointer");
  if (ld < 2 * F || ldo < F) FAIL("silu_mul: rows of %d for 2 x %d, output rows of %d", ld, F, ldo);
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("silu_mul: unknown dtype code %d", dtype);
  dim3 grid(n_rows, (F + 255) / 256), block(256);
  if (dtype == DT_F32) {
    if (activation)
      hipLaunchKernelGGL((silu_mul_kernel<float, true>), grid, block, 0, stream, (const float*)gu, ld, (float*)out, ldo, n_rows, F);
    else
      hipLaunchKernelGGL((silu_mul_kernel<float, false>), grid, block, 0, stream, (const float*)gu, ld, (float*)out, ldo, n_rows, F);
  } else {
    if (activation)
      hipLaunchKernelGGL((silu_mul_kernel<bf16, true>), grid, block, 0, stream, (const bf16*)gu, ld, (bf16*)out, ldo, n_rows, F);
    else
      hipLaunchKernelGGL((silu_mul_kernel<bf16, false>), grid, block, 0, stream, (const bf16*)gu, ld, (bf16*)out, ldo, n_rows, F);
  }
  CHECK_LAUNCH("silu_mul");
  return 0;
}

extern "C" int silu_mul(const void* gu, int ld, void* out, int ldo, int n_rows, int F, int dtype, hipStream_t stream) {
  return act_mul_launch(gu, ld, out, ldo, n_rows, F, dtype, 0, stream);
}

extern "C" int act_mul(const void* gu, int ld, void* out, int ldo, int n_rows, int F, int dtype, int activation,
                       hipStream_t stream) {
  return act_mul_launch(gu, ld, out, ldo, n_rows, F, dtype, activation, stream);
}

// act: [n_tokens * top, F] of the compute dtype; y: float rows.
extern "C" int expert_rows(const void* x, int ldx, const void* w_gate, const void* w_up, const void* w_down,
                           const int* idx, const float* weight, int n_tokens, int n_experts, int top, int F, int width,
                           void* act, float* y, int ldy, int accumulate, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (!x || !idx || !weight || !y || (n_experts > 0 && (!w_gate || !w_up || !w_down || !act)))
    FAIL("expert_rows: null pointer");
  if (top <= 0 || F <= 0 || width <= 0 || ldx < width || ldy < width) FAIL("expert_rows: sizes");
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("expert_rows: unknown dtype code %d", dtype);
  const int feats = 16, cols = 16, per = dtype == DT_BF16 ? 8 : 4;
  const bool vec = F % per == 0 && width % per == 0 && ldx % per == 0 && !((uintptr_t)x & 15);
  dim3 block(256), up_grid(n_tokens * top, (F + feats - 1) / feats), down_grid(n_tokens, (width + cols - 1) / cols);
#define RUN(T, VEC)                                                                                                        \
  do {                                                                                                                     \
    if (n_experts > 0)                                                                                                     \
      hipLaunchKernelGGL((expert_rows_up_kernel<T, VEC>), up_grid, block, 0, stream, (const T*)x, ldx, (const T*)w_gate,   \
                         (const T*)w_up, idx, weight, n_experts, top, F, width, (T*)act);                           \
    hipLaunchKernelGGL((expert_rows_down_kernel<T, VEC>), down_grid, block, 0, stream, (const T*)act, (const T*)w_down,    \
                       idx, weight, (const T*)x, ldx, n_experts, top, F, width, y, ldy, accumulate);                 \
  } while (0)
  if (dtype == DT_F32) {
    if (vec) RUN(float, true); else RUN(float, false);
  } else {
    if (vec) RUN(bf16, true); else RUN(bf16, false);
  }
#undef RUN
  CHECK_LAUNCH("expert_rows");
  return 0;
}

// The most tiles that n_items picks over n_experts experts can make.
extern "C" int expert_tiles_most(int n_items, int n_experts) { return (n_items + TILE_PICKS - 1) / TILE_PICKS + n_experts; }

// 1 if expert_tiles takes these sizes (the operands are read 16 bytes a lane).
extern "C" int expert_tiles_takes(int F, int width, int dtype) {
  const int kl = dtype == DT_BF16 ? 8 : 4;
  return F > 0 && F % kl == 0 && width % kl == 0;
}

// order: [n_tokens * top] ints, tiles: [3 * expert_tiles_most] ints, n_tiles: one int, act: [n_tokens * top, F]
// of the compute dtype, out: [n_tokens * top, width] floats.
extern "C" int expert_tiles(const void* x, int ldx, const void* w_gate, const void* w_up, const void* w_down, const int* idx,
                            const float* weight, int n_tokens, int n_experts, int top, int F, int width, int* order, int* tiles,
                            int* n_tiles, void* act, float* out, float* y, int ldy, int accumulate, int dtype,
                            hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (!x || !idx || !weight || !y || !w_gate || !w_up || !w_down || !order || !tiles || !n_tiles || !act || !out)
    FAIL("expert_tiles: null pointer");
  if (n_experts <= 0 || top <= 0 || ldx < width || ldy < width) FAIL("expert_tiles: sizes");
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("expert_tiles: unknown dtype code %d", dtype);
  if (!expert_tiles_takes(F, width, dtype)) FAIL("expert_tiles: inner size %d and width %d must be multiples of %d", F, width, dtype == DT_BF16 ? 8 : 4);
  if (n_experts > 8192) FAIL("expert_tiles: %d experts are more than the sorting block's LDS holds", n_experts);
  if (ldx % (dtype == DT_BF16 ? 8 : 4) || ((uintptr_t)x & 15)) FAIL("expert_tiles: the rows of x must be 16-byte aligned");
  const int n_items = n_tokens * top, most = expert_tiles_most(n_items, n_experts);
  hipLaunchKernelGGL(expert_sort_kernel, dim3(1), dim3(1024), 2 * n_experts * sizeof(int), stream, idx, n_items, n_experts,
                     order, tiles, n_tiles);
  // (wide blocks where the tiles alone fill the GPU, narrow ones where they are few)
  const bool wide = (long)most * ((F + 255) / 256) >= 256;
  const int per = wide ? 256 : 64;
  dim3 block(256), up_grid(most, (F + per - 1) / per), down_grid(most, (width + per - 1) / per), sum_grid(n_tokens, (width + 255) / 256);
#define RUN(T, CF)                                                                                                       \
  do {                                                                                                                   \
    hipLaunchKernelGGL((expert_tiles_up_kernel<T, CF>), up_grid, block, 0, stream, (const T*)x, ldx, (const T*)w_gate,   \
                       (const T*)w_up, order, tiles, n_tiles, weight, top, F, width, (T*)act);                           \
    hipLaunchKernelGGL((expert_tiles_down_kernel<T, CF>), down_grid, block, 0, stream, (const T*)act, (const T*)w_down,  \
                       order, tiles, n_tiles, F, width, out);                                                            \
    hipLaunchKernelGGL(expert_combine_kernel<T>, sum_grid, block, 0, stream, out, idx, weight, (const T*)x, ldx,         \
                       n_experts, top, width, y, ldy, accumulate);                                                       \
  } while (0)
  if (dtype == DT_F32) {
    if (wide) RUN(float, 4); else RUN(float, 1);
  } else {
    if (wide) RUN(bf16, 4); else RUN(bf16, 1);
  }
#undef RUN
  CHECK_LAUNCH("expert_tiles");
  return 0;
}
