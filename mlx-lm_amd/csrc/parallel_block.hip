// What a layer does around its sublayers when both read one norm of the stream and the stream
// that leaves the layer is a weighted sum of every earlier layer's result:
//
//   norm_fanout    h = x / sqrt(mean(x^2) + eps) * w  over the 32-bit stream x, a block a row, the
//                  row in registers: h in the compute dtype (what the feed-forward reads), h as
//                  floats (what a convolution over time reads), and up to two float copies of x
//                  itself (the row of the layers' results that the sublayers add into, and the
//                  embedding's row), each where its pointer is given.
//   depth_average  out[t] = sum_j a[j] * X_j[t] over the first n of the stacked results
//                  X [n_kept, tokens, width], all 32-bit.
#include "common.h"

template <typename T, int NV>
__global__ __launch_bounds__(256) void norm_fanout_kernel(const float* __restrict__ x, int ldx,
                                                          const float* __restrict__ gamma, float eps, int width,
                                                          T* __restrict__ out, float* __restrict__ out32,
                                                          float* __restrict__ copy_a, float* __restrict__ copy_b) {
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
  }
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

extern "C" int norm_fanout(const float* x, int ldx, const float* gamma, float eps, int n_rows, int width, void* out,
                           int out_dtype, float* out32, float* copy_a, float* copy_b, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!x || !gamma || !out) FAIL("norm_fanout: null pointer");
  if (width <= 0 || width % 4 || ldx < width || ldx % 4) FAIL("norm_fanout: rows of %d floats (stride %d), multiples of 4", width, ldx);
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) FAIL("norm_fanout: unknown dtype code %d", out_dtype);
  if ((((uintptr_t)x | (uintptr_t)gamma | (uintptr_t)out32 | (uintptr_t)copy_a | (uintptr_t)copy_b) & 15))
    FAIL("norm_fanout: 16-byte aligned rows");
  const dim3 grid(n_rows), block(256);
#define FANOUT(T, NV)                                                                                              \
  hipLaunchKernelGGL((norm_fanout_kernel<T, NV>), grid, block, 0, stream, x, ldx, gamma, eps, width, (T*)out, out32, \
                     copy_a, copy_b)
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
