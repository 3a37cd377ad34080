// Small 32-bit steps between a projection's float rows and a recurrence over them, and behind it:
//
//   silu_columns    u[t, c] <- silu(u[t, c]) for the columns [col, col + n) of float rows, in place
//                   (queries, keys and values of a linear attention that activates them).
//   forget_gate     a forget gate with a floor per channel, f = l + (1 - l) sigmoid(z), for a state
//                   S <- diag(f) S + (1 - f) v^T: the logits z (columns of float rows, bias added
//                   by the projection) become log f in place, and 1 - f = (1 - l) sigmoid(-z) goes to
//                   `keys`; queries in columns [q_col, q_col + n) pass a silu in place.
//   normed_gate     out = y / sqrt(mean(y^2) + eps) * w * sigmoid(g) over whole rows (all heads
//                   together), float rows in, the compute dtype out; a block a row.
#include "common.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

__global__ __launch_bounds__(256) void silu_columns_kernel(float* __restrict__ u, int ld, int col, int n) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= n) return;
  float* p = u + (size_t)blockIdx.x * ld + col + c;
  *p = silu_f(*p);
}

__global__ __launch_bounds__(256) void forget_gate_kernel(float* __restrict__ u, int ld, int q_col, int z_col, int n,
                                                          const float* __restrict__ lower, float* __restrict__ keys,
                                                          int ldk) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= n) return;
  float* row = u + (size_t)blockIdx.x * ld;
  const float z = row[z_col + c], l = lower[c];
  // 1 - f without cancellation; log f = log1p(-(1 - f)) keeps its digits where f is close to one,
  // log(l + (1 - l) sigmoid(z)) where it is small
  const float rest = (1.0f - l) / (1.0f + expf(z));
  row[z_col + c] = rest < 0.5f ? log1pf(-rest) : logf(l + (1.0f - l) / (1.0f + expf(-z)));
  keys[(size_t)blockIdx.x * ldk + c] = rest;
  row[q_col + c] = silu_f(row[q_col + c]);
}

template <typename T>
__global__ __launch_bounds__(256) void normed_gate_kernel(const float* __restrict__ y, int ldy, const float* __restrict__ g,
                                                          int ldg, const float* __restrict__ w, float eps, int width,
                                                          T* __restrict__ out, int ldo) {
  __shared__ float red[32];
  const int r = blockIdx.x;
  const float* yr = y + (size_t)r * ldy;
  float q = 0.f;
  for (int k = threadIdx.x; k < width; k += 256) q += yr[k] * yr[k];
  const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
  const float* gr = g + (size_t)r * ldg;
  for (int k = threadIdx.x; k < width; k += 256)
    out[(size_t)r * ldo + k] = from_f32<T>(yr[k] * rstd * w[k] / (1.0f + expf(-gr[k])));
}

DEFINE_LAST_ERROR(mlxlm_last_error)

extern "C" int silu_columns(float* u, int ld, int n_rows, int col, int n, hipStream_t stream) {
  if (n_rows <= 0 || n <= 0) return 0;
  if (!u || col < 0 || ld < col + n) FAIL("silu_columns: columns %d .. %d of rows of %d", col, col + n, ld);
  hipLaunchKernelGGL(silu_columns_kernel, dim3(n_rows, (n + 255) / 256), dim3(256), 0, stream, u, ld, col, n);
  CHECK_LAUNCH("silu_columns");
  return 0;
}

extern "C" int forget_gate(float* u, int ld, int n_rows, int q_col, int z_col, int n, const float* lower, float* keys,
                           int ldk, hipStream_t stream) {
  if (n_rows <= 0 || n <= 0) return 0;
  if (!u || !lower || !keys) FAIL("forget_gate: null pointer");
  if (q_col < 0 || z_col < 0 || ld < q_col + n || ld < z_col + n || ldk < n ||
      (q_col < z_col + n && z_col < q_col + n))
    FAIL("forget_gate: queries at %d and logits at %d, %d columns each, in rows of %d; keys in rows of %d", q_col, z_col,
         n, ld, ldk);
  hipLaunchKernelGGL(forget_gate_kernel, dim3(n_rows, (n + 255) / 256), dim3(256), 0, stream, u, ld, q_col, z_col, n,
                     lower, keys, ldk);
  CHECK_LAUNCH("forget_gate");
  return 0;
}

extern "C" int normed_gate(const float* y, int ldy, const float* g, int ldg, const float* w, float eps, int n_rows,
                           int width, void* out, int ldo, int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!y || !g || !w || !out) FAIL("normed_gate: null pointer");
  if (width <= 0 || ldy < width || ldg < width || ldo < width) FAIL("normed_gate: rows of %d in strides %d, %d, %d", width, ldy, ldg, ldo);
  if (out_dtype == DT_F32)
    hipLaunchKernelGGL(normed_gate_kernel<float>, dim3(n_rows), dim3(256), 0, stream, y, ldy, g, ldg, w, eps, width,
                       (float*)out, ldo);
  else if (out_dtype == DT_BF16)
    hipLaunchKernelGGL(normed_gate_kernel<bf16>, dim3(n_rows), dim3(256), 0, stream, y, ldy, g, ldg, w, eps, width,
                       (bf16*)out, ldo);
  else
    FAIL("normed_gate: unknown dtype code %d", out_dtype);
  CHECK_LAUNCH("normed_gate");
  return 0;
}
