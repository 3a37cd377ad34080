// What lies between a projection and the attention (or recurrence) that reads its heads, and
// between the attention and the output projection, for mixers that shape their heads in ways of
// their own.  Everything is 32-bit inside; the sources are the projections' float rows.
//
//   (causal convolution)  y[t, c] = sum_j w[c, j] u[t - taps + 1 + j, c] over a request's own tokens;
//                   inputs of earlier steps come from the request's state row ([taps - 1, C], the
//                   latest last, zero at a request's start), which conv_state_update
//                   (linear_state.hip) brings up to date afterwards.  With `conv_single` (every
//                   request brings one token) the kernel moves the state up itself.  It is an
//                   option of head_prepare: the source's columns pass through it on their way in.
//   head_prepare    a wave a (row, head): the head's `dim` columns from a float row (through the
//                   convolution, where one is given); RMS norm over
//                   the first `norm_dim` of them (or, with `norm_whole`, over all heads' columns at
//                   once, with a weight for each) (times a weight of norm_dim values shared by all
//                   heads, or none); rotation of the `rot_dims` columns from `rot_off` on by
//                   position * inv_freq[i], pairs (2i, 2i + 1) or (i, i + rot_dims / 2), cos and
//                   sin times `rot_mult`; then the head goes to `copies` places: copy c of head h
//                   to column dst_head[c * n_heads + h] * dst_stride of the output row (h itself
//                   without a table), zeros from `dim` up to `dst_fill` columns.  The output is
//                   rows of a matrix, or (block_table given) the pages of a cache: the row's
//                   request and position say which page and place, as kv_write has it.
//                   head_prepare_many: up to four such preparations in one launch.
//   diff_combine    o = a1 - lambda a2 per head, where a1 and a2 are two heads of an attention's
//                   output (tables say which), divided by its root mean square and multiplied by
//                   `mult`.
//   head_gate       x[t, h, :] *= sigmoid(g[t, h]), in place.
#include "common.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

#define PREPARE_CONV_MAX_DIM 256  // the widest head that passes a convolution

struct PrepareArgs {
  const float* src;
  int lds, src_col, src_stride;  // head h at column src_col + h * src_stride
  int n_rows, n_heads, dim;
  int norm_dim;
  const float* norm_w;  // [norm_dim] or null
  float eps;
  int rot_off, rot_dims, interleaved;
  const float* inv_freq;  // [rot_dims / 2]
  float rot_mult;
  const int* positions;
  void* dst;
  int ldd, dst_stride, dst_fill, copies;
  const int* dst_head;  // [copies, n_heads] or null
  // a causal convolution over the source's columns (column c of the row is channel c), or conv_w null
  const float* conv_w;  // [channels, taps]
  int taps, conv_channels, conv_single;
  float* conv_state;  // a request's row: [taps - 1, channels] at conv_offset, the latest last
  size_t conv_state_stride, conv_offset;
  const int* seq_start;  // [requests] the first row of a request in this step
  const int* slot_ids;   // [requests] its state row
  const int* token_req;  // [rows] (the convolution and the pages need it)
  // dst is a cache's pages (of dst_stride columns a head) where block_table is given
  const int* block_table;
  int max_blocks, page_size;
  size_t page_stride;
  // norm_whole > 0: the norm runs over the whole projection, the norm_whole columns from src_col
  // on (all heads at once), with a weight for every one of them (norm_w [norm_whole]); every
  // column of a head is normed.  Not together with a convolution.
  int norm_whole;
};

template <typename T>
__device__ __forceinline__ void prepare_head(const PrepareArgs& a, long item, int lane) {
  if (item >= (long)a.n_rows * a.n_heads) return;  // whole waves leave; no barrier follows
  const int row = (int)(item / a.n_heads), h = (int)(item % a.n_heads);
  const int first_col = a.src_col + h * a.src_stride;
  const float* s = a.src + (size_t)row * a.lds + first_col;
  const int req = (a.conv_w || a.block_table) ? a.token_req[row] : 0;
  const int local = a.conv_w ? row - a.seq_start[req] : 0;  // the row's place among its request's rows of this step
  float* old = a.conv_w ? a.conv_state + (size_t)a.slot_ids[req] * a.conv_state_stride + a.conv_offset : nullptr;
  // column c of the head as the rest sees it: as it is, or through the convolution (the oldest
  // input first), which is run once a column into the wave's own piece of LDS (the norm, the
  // column's own turn and its partner's read it)
  __shared__ float convolved[4][PREPARE_CONV_MAX_DIM];
  float* cv = convolved[threadIdx.x >> 6];
  if (a.conv_w) {
    for (int c = lane; c < a.dim; c += 64) {
      const int ch = first_col + c;
      float acc = 0.f;
      for (int j = a.taps - 1; j >= 0; --j) {
        const int at = local - j;
        const float u = at >= 0 ? s[c - (long)j * a.lds] : old[(size_t)(a.taps - 1 + at) * a.conv_channels + ch];
        acc += a.conv_w[(size_t)ch * a.taps + (a.taps - 1 - j)] * u;
      }
      cv[c] = acc;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // (the wave's lanes read each other's columns)
    __builtin_amdgcn_wave_barrier();
  }
  auto in = [&](int c) { return a.conv_w ? cv[c] : s[c]; };
  float rstd = 1.f;
  if (a.norm_whole > 0) {
    // (every wave of the row adds up the whole projection itself: a few loads a lane)
    const float* whole = a.src + (size_t)row * a.lds + a.src_col;
    float q = 0.f;
    for (int k = lane; k < a.norm_whole; k += 64) q += whole[k] * whole[k];
    rstd = 1.0f / sqrtf(wave_sum(q) / (float)a.norm_whole + a.eps);
  } else if (a.norm_dim > 0) {
    float q = 0.f;
    for (int k = lane; k < a.norm_dim; k += 64) {
      const float u = in(k);
      q += u * u;
    }
    rstd = 1.0f / sqrtf(wave_sum(q) / (float)a.norm_dim + a.eps);
  }
  const int position = (a.rot_dims || a.block_table) ? a.positions[row] : 0;
  const float pos = (float)position;
  const int half = a.rot_dims / 2;
  // where head dh of this row starts in dst
  const size_t page_base = a.block_table ? (size_t)a.block_table[(size_t)req * a.max_blocks + position / a.page_size] * a.page_stride : 0;
  auto head_at = [&](int dh) {
    return a.block_table ? page_base + ((size_t)dh * a.page_size + position % a.page_size) * a.dst_stride
                         : (size_t)row * a.ldd + (size_t)dh * a.dst_stride;
  };
  for (int k = lane; k < a.dst_fill; k += 64) {
    float v = 0.f;
    if (k < a.dim) {
      const int rel = k - a.rot_off;
      auto at = [&](int c) {
        if (a.norm_whole > 0) return in(c) * rstd * (a.norm_w ? a.norm_w[h * a.src_stride + c] : 1.f);
        return c < a.norm_dim ? in(c) * rstd * (a.norm_w ? a.norm_w[c] : 1.f) : in(c);
      };
      v = at(k);
      if (rel >= 0 && rel < a.rot_dims) {
        int i, partner;
        bool first;  // this column is the pair's first member
        if (a.interleaved)
          i = rel >> 1, first = !(rel & 1), partner = first ? k + 1 : k - 1;
        else
          first = rel < half, i = first ? rel : rel - half, partner = first ? k + half : k - half;
        float sn, cs;
        sincosf(pos * a.inv_freq[i], &sn, &cs);
        sn *= a.rot_mult, cs *= a.rot_mult;
        const float other = at(partner);
        v = first ? v * cs - other * sn : v * cs + other * sn;
      }
    }
    for (int c = 0; c < a.copies; ++c) {
      const int dh = a.dst_head ? a.dst_head[c * a.n_heads + h] : h;
      ((T*)a.dst)[head_at(dh) + k] = from_f32<T>(v);
    }
  }
  if (a.conv_w && a.conv_single && a.taps > 1) {
    // every request brings one token: this wave alone reads and writes its request's inputs of this
    // head's channels, so it moves them up by one itself, after everything above has been read
    // (a lane read its neighbours' channels for the rotation: the wave's loads are waited for first)
    __builtin_amdgcn_s_waitcnt(0);
    for (int k = lane; k < a.dim; k += 64) {
      const int ch = first_col + k;
      for (int j = 0; j + 2 < a.taps; ++j) old[(size_t)j * a.conv_channels + ch] = old[(size_t)(j + 1) * a.conv_channels + ch];
      old[(size_t)(a.taps - 2) * a.conv_channels + ch] = s[k];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void head_prepare_kernel(PrepareArgs a) {
  prepare_head<T>(a, (long)blockIdx.x * 4 + (threadIdx.x >> 6), threadIdx.x & 63);
}

// Several preparations in one launch (a mixer's queries, keys and values): the blocks of each
// follow those of the one before.
#define PREPARE_MOST 4
struct PrepareMany {
  PrepareArgs seg[PREPARE_MOST];
  unsigned first_block[PREPARE_MOST + 1];
  int n;
};

template <typename T>
__global__ __launch_bounds__(256) void head_prepare_many_kernel(PrepareMany m) {
  int s = 0;
  while (s + 1 < m.n && blockIdx.x >= m.first_block[s + 1]) ++s;
  prepare_head<T>(m.seg[s], (long)(blockIdx.x - m.first_block[s]) * 4 + (threadIdx.x >> 6), threadIdx.x & 63);
}

// A wave a (row, head).
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(const T* __restrict__ att, int lda, int head_stride,
                                                           const int* __restrict__ first, const int* __restrict__ second,
                                                           float lambda, float mult, float eps, int n_rows, int n_heads,
                                                           int vdim, T* __restrict__ out, int ldo) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long)n_rows * n_heads) return;
  const int row = (int)(item / n_heads), h = (int)(item % n_heads);
  const T* a1 = att + (size_t)row * lda + (size_t)first[h] * head_stride;
  const T* a2 = att + (size_t)row * lda + (size_t)second[h] * head_stride;
  float q = 0.f;
  for (int k = lane; k < vdim; k += 64) {
    const float o = to_f32(a1[k]) - lambda * to_f32(a2[k]);
    q += o * o;
  }
  const float f = mult / sqrtf(wave_sum(q) / (float)vdim + eps);
  for (int k = lane; k < vdim; k += 64)
    out[(size_t)row * ldo + (size_t)h * vdim + k] = from_f32<T>((to_f32(a1[k]) - lambda * to_f32(a2[k])) * f);
}

// Thread (row, column).
template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(T* __restrict__ x, int ldx, int head_stride, int n_heads,
                                                        const float* __restrict__ g, int ldg, int n_rows) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  const int width = n_heads * head_stride;
  if (e >= (long)n_rows * width) return;
  const int row = (int)(e / width), c = (int)(e % width);
  const float z = g[(size_t)row * ldg + c / head_stride];
  T* p = x + (size_t)row * ldx + c;
  *p = from_f32<T>(to_f32(*p) / (1.0f + expf(-z)));
}

DEFINE_LAST_ERROR(mlxlm_last_error)

static int prepare_args_fit(const PrepareArgs& a) {
  if (!a.src || !a.dst) FAIL("head_prepare: null pointer");
  if (a.dim <= 0 || a.src_col < 0 || a.src_col + (long)(a.n_heads - 1) * a.src_stride + a.dim > a.lds)
    FAIL("head_prepare: %d heads of %d columns, %d apart from column %d, in rows of %d", a.n_heads, a.dim, a.src_stride,
         a.src_col, a.lds);
  if (a.norm_dim < 0 || a.norm_dim > a.dim) FAIL("head_prepare: a norm over %d of %d columns", a.norm_dim, a.dim);
  if (a.norm_whole < 0 || (a.norm_whole > 0 && (a.conv_w || a.norm_whole < (a.n_heads - 1) * a.src_stride + a.dim ||
                                                 a.lds < a.src_col + a.norm_whole)))
    FAIL("head_prepare: a norm over the whole projection of %d columns (no convolution; all heads inside)", a.norm_whole);
  if (a.rot_dims && (a.rot_dims % 2 || a.rot_off < 0 || a.rot_off + a.rot_dims > a.dim || !a.inv_freq || !a.positions))
    FAIL("head_prepare: %d turning columns from %d in a head of %d", a.rot_dims, a.rot_off, a.dim);
  if (a.copies < 1 || a.dst_fill < a.dim || a.dst_fill > a.dst_stride)
    FAIL("head_prepare: %d copies, %d columns filled of %d, a head of %d", a.copies, a.dst_fill, a.dst_stride, a.dim);
  if (!a.block_table && !a.dst_head && (a.copies != 1 || (long)(a.n_heads - 1) * a.dst_stride + a.dst_fill > a.ldd))
    FAIL("head_prepare: the heads do not fit rows of %d", a.ldd);
  if (a.conv_w && a.dim > PREPARE_CONV_MAX_DIM) FAIL("head_prepare: heads of %d columns through a convolution (at most %d)", a.dim, PREPARE_CONV_MAX_DIM);
  if (a.conv_w && (a.taps < 1 || a.conv_channels < a.src_col + (a.n_heads - 1) * a.src_stride + a.dim || !a.conv_state ||
                   !a.seq_start || !a.slot_ids || !a.token_req))
    FAIL("head_prepare: a convolution of %d taps over %d channels needs its state and the rows' requests", a.taps, a.conv_channels);
  if (a.block_table && (!a.token_req || !a.positions || a.max_blocks <= 0 || a.page_size <= 0 || a.dst_fill != a.dst_stride))
    FAIL("head_prepare: pages of %d places need the rows' requests and positions, and whole heads of %d columns", a.page_size, a.dst_stride);
  return 0;
}

extern "C" int head_prepare(const PrepareArgs* args, int dst_dtype, hipStream_t stream) {
  const PrepareArgs& a = *args;
  if (a.n_rows <= 0 || a.n_heads <= 0) return 0;
  if (prepare_args_fit(a)) return 1;
  if (dst_dtype != DT_F32 && dst_dtype != DT_BF16) FAIL("head_prepare: unknown dtype code %d", dst_dtype);
  const long items = (long)a.n_rows * a.n_heads;
  dim3 grid((unsigned)((items + 3) / 4)), block(256);
  if (dst_dtype == DT_F32)
    hipLaunchKernelGGL(head_prepare_kernel<float>, grid, block, 0, stream, a);
  else
    hipLaunchKernelGGL(head_prepare_kernel<bf16>, grid, block, 0, stream, a);
  CHECK_LAUNCH("head_prepare");
  return 0;
}

// `n` preparations (1 to 4) whose outputs are all of `dst_dtype`, in one launch.
extern "C" int head_prepare_many(const PrepareArgs* args, int n, int dst_dtype, hipStream_t stream) {
  if (n < 1 || n > PREPARE_MOST || !args) FAIL("head_prepare_many: %d preparations (1 to %d)", n, PREPARE_MOST);
  if (dst_dtype != DT_F32 && dst_dtype != DT_BF16) FAIL("head_prepare: unknown dtype code %d", dst_dtype);
  PrepareMany m;
  m.n = 0;
  unsigned blocks = 0;
  for (int i = 0; i < n; ++i) {
    const PrepareArgs& a = args[i];
    if (a.n_rows <= 0 || a.n_heads <= 0) continue;
    if (prepare_args_fit(a)) return 1;
    m.seg[m.n] = a, m.first_block[m.n] = blocks;
    blocks += (unsigned)(((long)a.n_rows * a.n_heads + 3) / 4);
    ++m.n;
  }
  if (m.n == 0) return 0;
  for (int i = m.n; i <= PREPARE_MOST; ++i) m.first_block[i] = blocks;
  if (dst_dtype == DT_F32)
    hipLaunchKernelGGL(head_prepare_many_kernel<float>, dim3(blocks), dim3(256), 0, stream, m);
  else
    hipLaunchKernelGGL(head_prepare_many_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, m);
  CHECK_LAUNCH("head_prepare_many");
  return 0;
}

extern "C" int diff_combine(const void* att, int lda, int head_stride, const int* first, const int* second, float lambda,
                            float mult, float eps, int n_rows, int n_heads, int vdim, void* out, int ldo, int dtype,
                            hipStream_t stream) {
  if (n_rows <= 0 || n_heads <= 0) return 0;
  if (!att || !first || !second || !out) FAIL("diff_combine: null pointer");
  if (vdim <= 0 || vdim > head_stride || ldo < n_heads * vdim) FAIL("diff_combine: values of %d in heads of %d, rows of %d", vdim, head_stride, ldo);
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("diff_combine: unknown dtype code %d", dtype);
  const long items = (long)n_rows * n_heads;
  dim3 grid((unsigned)((items + 3) / 4)), block(256);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(diff_combine_kernel<float>, grid, block, 0, stream, (const float*)att, lda, head_stride, first, second,
                       lambda, mult, eps, n_rows, n_heads, vdim, (float*)out, ldo);
  else
    hipLaunchKernelGGL(diff_combine_kernel<bf16>, grid, block, 0, stream, (const bf16*)att, lda, head_stride, first, second,
                       lambda, mult, eps, n_rows, n_heads, vdim, (bf16*)out, ldo);
  CHECK_LAUNCH("diff_combine");
  return 0;
}

extern "C" int head_gate(void* x, int ldx, int head_stride, int n_heads, const float* g, int ldg, int n_rows, int dtype,
                         hipStream_t stream) {
  if (n_rows <= 0 || n_heads <= 0) return 0;
  if (!x || !g) FAIL("head_gate: null pointer");
  if (head_stride <= 0 || ldx < n_heads * head_stride || ldg < n_heads)
    FAIL("head_gate: %d heads of %d columns in rows of %d, gates in rows of %d", n_heads, head_stride, ldx, ldg);
  if (dtype != DT_F32 && dtype != DT_BF16) FAIL("head_gate: unknown dtype code %d", dtype);
  const long total = (long)n_rows * n_heads * head_stride;
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (dtype == DT_F32)
    hipLaunchKernelGGL(head_gate_kernel<float>, grid, block, 0, stream, (float*)x, ldx, head_stride, n_heads, g, ldg, n_rows);
  else
    hipLaunchKernelGGL(head_gate_kernel<bf16>, grid, block, 0, stream, (bf16*)x, ldx, head_stride, n_heads, g, ldg, n_rows);
  CHECK_LAUNCH("head_gate");
  return 0;
}
