// What a layer does around its sublayers when both read one norm of the stream and the stream
// that leaves the layer is a weighted sum of every earlier layer's result:
//
//   norm_fanout    h = x / sqrt(mean(x^2) + eps) * w  over the 32-bit stream x, a block a row, the
//                  row in registers: h in the compute dtype (what the feed-forward reads), h as
//                  floats (what a convolution over time reads), and up to two float copies of x
//                  itself (the row of the layers' results that the sublayers add into, and the
//                  embedding's row), each where its pointer is given.
//                  With `canon` (a step in which every request brings one token) the kernel also
//                  runs the causal convolution over time that the mixer's input passes,
//                  m = h + sum_j w[:, j] h_(t - taps + 1 + j), against the request's last taps - 1
//                  normed rows in its state row, and moves those up by one.
//   canon_rows     the same convolution for steps of any shape: float rows h of this step in, the
//                  compute dtype out; rows ahead of a request's first of this step come from its
//                  state row ([taps - 1, width], the latest last), which conv_state_update
//                  (linear_state.hip) brings up to date afterwards.
//   depth_average  out[t] = sum_j a[j] * X_j[t] over the first n of the stacked results
//                  X [n_kept, tokens, width], all 32-bit.
#include "common.h"

// The convolution over time on a mixer's input: weights [width, taps] (the last tap meets the
// current token), a request's state row holding its last taps - 1 inputs from state_offset on.
struct CanonArgs {
  const float* w;
  int taps;
  float* state;
  size_t state_stride, state_offset;
  const int* token_req;  // [rows]
  const int* seq_start;  // [requests] the first row of a request in this step (canon_rows)
  const int* slot_ids;   // [requests] its state row
  void* mixed;           // [rows, width] out, the compute dtype
};

template <typename T, int NV, bool CANON>
__global__ __launch_bounds__(256) void norm_fanout_kernel(const float* __restrict__ x, int ldx,
                                                          const float* __restrict__ gamma, float eps, int width,
                                                          T* __restrict__ out, float* __restrict__ out32,
                                                          float* __restrict__ copy_a, float* __restrict__ copy_b,
                                                          CanonArgs cn) {
  __shared__ float red[32];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* xr = x + (size_t)r * ldx;
  float4 v[NV], g[NV];
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = min((tid + 256 * i) * 4, width - 4);
    v[i] = *(const float4*)(xr + k);
    g[i] = *(const float4*)(gamma + k);
  }
#pragma unroll
  for (int i = 0; i < NV; ++i)
    if ((tid + 256 * i) * 4 < width) q += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
  const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = (tid + 256 * i) * 4;
    if (k >= width) continue;
    const size_t at = (size_t)r * width + k;
    const float4 h = make_float4(v[i].x * rstd * g[i].x, v[i].y * rstd * g[i].y, v[i].z * rstd * g[i].z,
                                 v[i].w * rstd * g[i].w);
    T* o = out + at;
    o[0] = from_f32<T>(h.x), o[1] = from_f32<T>(h.y), o[2] = from_f32<T>(h.z), o[3] = from_f32<T>(h.w);
    if (out32) *(float4*)(out32 + at) = h;
    if (copy_a) *(float4*)(copy_a + at) = v[i];
    if (copy_b) *(float4*)(copy_b + at) = v[i];
    if constexpr (CANON) {
      // this row is its request's only one: the thread owns these four channels of the state row
      float* old = cn.state + (size_t)cn.slot_ids[cn.token_req[r]] * cn.state_stride + cn.state_offset + k;
      const float hv[4] = {h.x, h.y, h.z, h.w};
      float m[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) m[c] = hv[c] + cn.w[(size_t)(k + c) * cn.taps + cn.taps - 1] * hv[c];
      // (a state row may start anywhere: a float at a time)
      for (int j = 0; j + 1 < cn.taps; ++j) {
        float ov[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) ov[c] = old[(size_t)j * width + c];
#pragma unroll
        for (int c = 0; c < 4; ++c) m[c] += cn.w[(size_t)(k + c) * cn.taps + j] * ov[c];
        if (j > 0) {
#pragma unroll
          for (int c = 0; c < 4; ++c) old[(size_t)(j - 1) * width + c] = ov[c];
        }
      }
      if (cn.taps > 1) {
#pragma unroll
        for (int c = 0; c < 4; ++c) old[(size_t)(cn.taps - 2) * width + c] = hv[c];
      }
      T* mo = (T*)cn.mixed + at;
      mo[0] = from_f32<T>(m[0]), mo[1] = from_f32<T>(m[1]), mo[2] = from_f32<T>(m[2]), mo[3] = from_f32<T>(m[3]);
    }
  }
}

// A thread four channels of a row: the row's own normed values and the taps - 1 before it, from
// this step's rows or, ahead of the request's first row of this step, from its state row.
template <typename T>
__global__ __launch_bounds__(256) void canon_rows_kernel(const float* __restrict__ h, int width, CanonArgs cn) {
  const int r = blockIdx.x, k = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (k >= width) return;
  const int req = cn.token_req[r];
  const int local = r - cn.seq_start[req];
  const float* old = cn.state + (size_t)cn.slot_ids[req] * cn.state_stride + cn.state_offset + k;
  const float4 cur = *(const float4*)(h + (size_t)r * width + k);
  const float hv[4] = {cur.x, cur.y, cur.z, cur.w};
  float m[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) m[c] = hv[c] + cn.w[(size_t)(k + c) * cn.taps + cn.taps - 1] * hv[c];
  for (int j = 0; j + 1 < cn.taps; ++j) {
    const int back = cn.taps - 1 - j;  // how many tokens before this one
    const float* o = local >= back ? h + (size_t)(r - back) * width + k : old + (size_t)(cn.taps - 1 + local - back) * width;
    const float ov[4] = {o[0], o[1], o[2], o[3]};  // (a state row may start anywhere: a float at a time)
#pragma unroll
    for (int c = 0; c < 4; ++c) m[c] += cn.w[(size_t)(k + c) * cn.taps + j] * ov[c];
  }
  T* mo = (T*)cn.mixed + (size_t)r * width + k;
  mo[0] = from_f32<T>(m[0]), mo[1] = from_f32<T>(m[1]), mo[2] = from_f32<T>(m[2]), mo[3] = from_f32<T>(m[3]);
}

// Any width that is a multiple of 4 beyond what a block keeps in registers: the row read twice.
template <typename T>
__global__ __launch_bounds__(256) void norm_fanout_wide_kernel(const float* __restrict__ x, int ldx,
                                                               const float* __restrict__ gamma, float eps, int width,
                                                               T* __restrict__ out, float* __restrict__ out32,
                                                               float* __restrict__ copy_a, float* __restrict__ copy_b) {
  __shared__ float red[32];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* xr = x + (size_t)r * ldx;
  float q = 0.f;
  for (int k = tid; k < width; k += 256) q += xr[k] * xr[k];
  const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
  for (int k = tid; k < width; k += 256) {
    const size_t at = (size_t)r * width + k;
    const float h = xr[k] * rstd * gamma[k];
    out[at] = from_f32<T>(h);
    if (out32) out32[at] = h;
    if (copy_a) copy_a[at] = xr[k];
    if (copy_b) copy_b[at] = xr[k];
  }
}

#define DEPTH_MAX 256  // the most results a sum takes (its weights travel in LDS)

__global__ __launch_bounds__(256) void depth_average_kernel(float* __restrict__ out, const float* __restrict__ kept,
                                                            size_t stride, const float* __restrict__ a, int n,
                                                            size_t n_vec) {
  __shared__ float w[DEPTH_MAX];
  for (int j = threadIdx.x; j < n; j += 256) w[j] = a[j];
  __syncthreads();
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_vec) return;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int j = 0; j < n; ++j) {
    const float4 v = *(const float4*)(kept + (size_t)j * stride + 4 * i);
    s.x += w[j] * v.x, s.y += w[j] * v.y, s.z += w[j] * v.z, s.w += w[j] * v.w;
  }
  *(float4*)(out + 4 * i) = s;
}

DEFINE_LAST_ERROR(mlxlm_last_error)

static int check_canon(const char* who, const CanonArgs* cn, int width, bool rows) {
  if (!cn->w || !cn->state || !cn->token_req || !cn->slot_ids || !cn->mixed || (rows && !cn->seq_start))
    FAIL("%s: the convolution's pointers", who);
  if (cn->taps < 1 || cn->state_stride < cn->state_offset + (size_t)(cn->taps - 1) * width)
    FAIL("%s: %d taps over %d channels do not fit state rows of %zu floats from %zu on", who, cn->taps, width,
         cn->state_stride, cn->state_offset);
  return 0;
}

// `canon` (or null): every row is its request's only one of this step; the convolution runs here
// too, and the requests' state rows move up by one.
extern "C" int norm_fanout(const float* x, int ldx, const float* gamma, float eps, int n_rows, int width, void* out,
                           int out_dtype, float* out32, float* copy_a, float* copy_b, const CanonArgs* canon,
                           hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (canon && check_canon("norm_fanout", canon, width, false)) return 1;
  if (canon && width > 8192) FAIL("norm_fanout: the convolution rides along up to 8192 columns, not %d", width);
  const CanonArgs cn = canon ? *canon : CanonArgs{};
  if (!x || !gamma || !out) FAIL("norm_fanout: null pointer");
  if (width <= 0 || width % 4 || ldx < width || ldx % 4) FAIL("norm_fanout: rows of %d floats (stride %d), multiples of 4", width, ldx);
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) FAIL("norm_fanout: unknown dtype code %d", out_dtype);
  if ((((uintptr_t)x | (uintptr_t)gamma | (uintptr_t)out32 | (uintptr_t)copy_a | (uintptr_t)copy_b) & 15))
    FAIL("norm_fanout: 16-byte aligned rows");
  const dim3 grid(n_rows), block(256);
#define FANOUT(T, NV)                                                                                                  \
  do {                                                                                                                 \
    if (canon)                                                                                                         \
      hipLaunchKernelGGL((norm_fanout_kernel<T, NV, true>), grid, block, 0, stream, x, ldx, gamma, eps, width, (T*)out, \
                         out32, copy_a, copy_b, cn);                                                                   \
    else                                                                                                               \
      hipLaunchKernelGGL((norm_fanout_kernel<T, NV, false>), grid, block, 0, stream, x, ldx, gamma, eps, width, (T*)out, \
                         out32, copy_a, copy_b, cn);                                                                   \
  } while (0)
#define FANOUT_BY_WIDTH(T)                                                                                  \
  if (width <= 1024) FANOUT(T, 1);                                                                          \
  else if (width <= 2048) FANOUT(T, 2);                                                                     \
  else if (width <= 4096) FANOUT(T, 4);                                                                     \
  else if (width <= 8192) FANOUT(T, 8);                                                                     \
  else hipLaunchKernelGGL(norm_fanout_wide_kernel<T>, grid, block, 0, stream, x, ldx, gamma, eps, width, (T*)out, \
                          out32, copy_a, copy_b)
  if (out_dtype == DT_F32) {
    FANOUT_BY_WIDTH(float);
  } else {
    FANOUT_BY_WIDTH(bf16);
  }
#undef FANOUT_BY_WIDTH
#undef FANOUT
  CHECK_LAUNCH("norm_fanout");
  return 0;
}

extern "C" int canon_rows(const float* h, int n_rows, int width, int out_dtype, const CanonArgs* canon, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!h || !canon) FAIL("canon_rows: null pointer");
  if (width <= 0 || width % 4 || ((uintptr_t)h & 15)) FAIL("canon_rows: rows of %d floats, a multiple of 4, 16-byte aligned", width);
  if (check_canon("canon_rows", canon, width, true)) return 1;
  const dim3 grid(n_rows, (width / 4 + 255) / 256), block(256);
  if (out_dtype == DT_F32)
    hipLaunchKernelGGL(canon_rows_kernel<float>, grid, block, 0, stream, h, width, *canon);
  else if (out_dtype == DT_BF16)
    hipLaunchKernelGGL(canon_rows_kernel<bf16>, grid, block, 0, stream, h, width, *canon);
  else
    FAIL("canon_rows: unknown dtype code %d", out_dtype);
  CHECK_LAUNCH("canon_rows");
  return 0;
}

extern "C" int depth_average(float* out, const float* kept, size_t stride, const float* a, int n, int n_rows, int width,
                             hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!out || !kept || !a) FAIL("depth_average: null pointer");
  if (n <= 0 || n > DEPTH_MAX) FAIL("depth_average: a sum of %d results, 1 to %d", n, DEPTH_MAX);
  if (width <= 0 || width % 4 || stride % 4 || stride < (size_t)n_rows * width)
    FAIL("depth_average: %d rows of %d floats, results %zu floats apart", n_rows, width, stride);
  if (((uintptr_t)out | (uintptr_t)kept) & 15) FAIL("depth_average: 16-byte aligned rows");
  const size_t n_vec = (size_t)n_rows * width / 4;
  hipLaunchKernelGGL(depth_average_kernel, dim3((unsigned)((n_vec + 255) / 256)), dim3(256), 0, stream, out, kept, stride,
                     a, n, n_vec);
  CHECK_LAUNCH("depth_average");
  return 0;
}
