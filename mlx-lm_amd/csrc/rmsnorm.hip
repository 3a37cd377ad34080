// RMS norm over the last axis of the 32-bit residual stream:
//   y = x / sqrt(mean(x^2) + eps) * gamma          (eps inside the root; gamma may be absent)
// The mean of squares, the root and the scale are computed in 32-bit; the output is float or
// bfloat16.  With `rows` given, output row r is made from input row rows[r] (the rows whose
// logits are wanted).  A block a row with the row in registers; a wave a row for odd widths.
//
// Also the native part that stands for such a norm in a model (engine_parts.h).
#include "common.h"
#include "engine_parts.h"

// A block a row, the row in registers (NV float4 a thread, width <= 1024 NV): one trip to memory.
template <typename T, int NV>
__global__ __launch_bounds__(256) void rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ x, int ldx,
                                                      const int* __restrict__ rows, const float* __restrict__ gamma,
                                                      float eps, int width) {
  __shared__ float red[32];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * ldx;
  float4 v[NV], g[NV];
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = min((tid + 256 * i) * 4, width - 4);
    v[i] = *(const float4*)(xr + k);
    g[i] = gamma ? *(const float4*)(gamma + k) : make_float4(1.f, 1.f, 1.f, 1.f);
  }
#pragma unroll
  for (int i = 0; i < NV; ++i)
    if ((tid + 256 * i) * 4 < width) q += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
  const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int k = (tid + 256 * i) * 4;
    if (k >= width) continue;
    T* o = out + (size_t)r * width + k;
    o[0] = from_f32<T>(v[i].x * rstd * g[i].x), o[1] = from_f32<T>(v[i].y * rstd * g[i].y);
    o[2] = from_f32<T>(v[i].z * rstd * g[i].z), o[3] = from_f32<T>(v[i].w * rstd * g[i].w);
  }
}

// Any width and alignment: a wave a row, a column a lane at a time, the row read twice.
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_any_kernel(T* __restrict__ out, const float* __restrict__ x, int ldx,
                                                          const int* __restrict__ rows, const float* __restrict__ gamma,
                                                          float eps, int n_rows, int width) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;  // whole waves leave; no barrier follows
  const float* xr = x + (size_t)(rows ? rows[r] : r) * ldx;
  float q = 0.f;
  for (int k = lane; k < width; k += 64) q += xr[k] * xr[k];
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
  T* o = out + (size_t)r * width;
  for (int k = lane; k < width; k += 64) o[k] = from_f32<T>(xr[k] * rstd * (gamma ? gamma[k] : 1.f));
}

DEFINE_LAST_ERROR(mlxlm_last_error)

extern "C" int rmsnorm(void* out, const float* x, int ldx, const int* rows, const float* gamma, float eps, int n_rows,
                       int width, int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || ldx < width) FAIL("rmsnorm: width %d, row stride %d", width, ldx);
  if (!out || !x) FAIL("rmsnorm: null pointer");
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) FAIL("rmsnorm: unknown dtype code %d", out_dtype);
  const int nv4 = (width / 4 + 255) / 256;
  const int nv = nv4 <= 1 ? 1 : nv4 <= 2 ? 2 : nv4 <= 4 ? 4 : nv4 <= 8 ? 8 : 0;
  const bool vec = nv > 0 && width % 4 == 0 && ldx % 4 == 0 && !(((uintptr_t)x | (uintptr_t)gamma) & 15);
  if (vec) {
#define LAUNCH(T, NV) \
  hipLaunchKernelGGL((rmsnorm_kernel<T, NV>), dim3(n_rows), dim3(256), 0, stream, (T*)out, x, ldx, rows, gamma, eps, width)
#define BY_VECTORS(T)            \
  do {                           \
    if (nv == 1) LAUNCH(T, 1);   \
    else if (nv == 2) LAUNCH(T, 2); \
    else if (nv == 4) LAUNCH(T, 4); \
    else LAUNCH(T, 8);           \
  } while (0)
    if (out_dtype == DT_F32)
      BY_VECTORS(float);
    else
      BY_VECTORS(bf16);
#undef BY_VECTORS
#undef LAUNCH
  } else {
    dim3 grid((n_rows + 3) / 4), block(256);
    if (out_dtype == DT_F32)
      hipLaunchKernelGGL(rmsnorm_any_kernel<float>, grid, block, 0, stream, (float*)out, x, ldx, rows, gamma, eps, n_rows, width);
    else
      hipLaunchKernelGGL(rmsnorm_any_kernel<bf16>, grid, block, 0, stream, (bf16*)out, x, ldx, rows, gamma, eps, n_rows, width);
  }
  CHECK_LAUNCH("rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------
// the part

static const EngHost* host = nullptr;

struct RmsNorm : Norm {
  int width;
  float eps;
  const float* gamma;
  RmsNorm(int w, float e, const float* g) : width(w), eps(e), gamma(g) {}
  int forward(EngCtx* ctx, const EngMat& x, const int* rows, int n_rows, bool lazy, const EngWeight*, bool,
              EngValue* out) override {
    if (x.cols != width || x.dtype != DT_F32) return host->fail("rmsnorm: float32 rows of width %d", width);
    *out = EngValue{};
    if (lazy && !rows) {
      // the consumer's first matrix product may norm the rows itself (lazy 2: no mean, no shift)
      out->lazy = 2, out->x = (const float*)x.p, out->ldx = x.ld, out->gamma = gamma, out->beta = nullptr;
      out->eps = eps;
      out->m = EngMat{nullptr, x.rows, width, width, ctx->dtype};
      return 0;
    }
    if (host->take(ctx, rows ? n_rows : x.rows, width, ctx->dtype, &out->m)) return 1;
    if (rmsnorm(out->m.p, (const float*)x.p, x.ld, rows, gamma, eps, out->m.rows, width, ctx->dtype, ctx->stream))
      return host->fail("%s", g_err);
    host->launched(ctx);
    return 0;
  }
};

extern "C" EngPart* make_rmsnorm(const EngHost* h, int width, float eps, const float* gamma) {
  host = h;
  return new RmsNorm(width, eps, gamma);
}
