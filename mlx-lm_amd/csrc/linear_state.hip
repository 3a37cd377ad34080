// Mixers whose memory of a sequence is a matrix per head that decays and takes an outer product
// at every token (linear attention with a decay, the selective state space with a scalar decay a
// head), and the kernels around them:
//
//   state_scan      S_t = a_t S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t  (+ skip_h v_t)
//                   S is N x P (key size x value size), 32-bit, kept per request and head between
//                   steps.  a_t = exp(log_a[t, h]) or the constant decay[h]; k_t is multiplied by
//                   k_mult and by k_scale[t, h] where given; q and k may turn with the position
//                   (the first rot_dims columns of a head, column i with column i + rot_dims / 2,
//                   by position * inv_freq[i]; the kernels that take chunks turn q and k in place
//                   first, so the caller must not need them afterwards); the key heads may be fewer than the value heads
//                   (head h reads key head h / (H / Hk)).  The output may be divided by its root
//                   mean square over the head and multiplied by silu(gate) on the way out.
//   ssm_prepare     causal convolution per channel over a request's tokens with the last
//                   taps - 1 inputs of earlier steps from the state, bias, silu; and the step
//                   sizes: dt = softplus(raw + dt_bias), log_a = -exp(A_log) dt.
//   conv_state_update  the last taps - 1 inputs of each request, for the next step.
//   gated_group_rmsnorm  out = RMSnorm_in_groups(y * silu(z)) * w.
//
// Everything here is 32-bit: the operands arrive as float rows (the projections write float),
// the state is float, angles, decays, exponentials and norms are float; only `out` of the scan
// and of the gated norm may be bfloat16.  Sums run in a fixed order.
#include "common.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

struct ScanArgs {
  const float* q;
  const float* k;
  const float* v;
  int ldq, ldk, ldv;
  const float* log_a;    // [tokens, H] or null
  const float* decay;    // [H], where log_a is null
  const float* k_scale;  // [tokens, H] or null
  float k_mult;
  const float* skip;  // [H] or null
  int rot_dims;
  const float* inv_freq;  // [rot_dims / 2]
  const int* positions;   // [tokens]
  int unit_rms;
  float eps;
  const float* gate;  // [tokens, ldg] or null, head h at column h * P
  int ldg;
  void* out;  // [tokens, ldo], head h at column h * P
  int ldo, out_dtype;
  float* state;  // request r, head h: state + slot_ids[r] * state_stride + state_offset + h * N * P
  size_t state_stride, state_offset;
  const int* seq_start;
  const int* seq_len;
  const int* slot_ids;
  int n_requests, H, Hk, N, P;
  int n_tokens_hint;  // the token rows of q and k (the kernels that take chunks turn them all at once, in place)
  // A decay per key channel instead of one a head: chan_a [tokens, ldca], head h at column h * N,
  // holds log a (<= 0), or, with chan_logit, a logit z with log a = chan_mult * log sigmoid(z).
  const float* chan_a;
  int ldca, chan_logit;
  float chan_mult;
  const float* norm_w;  // [P] or null: with unit_rms, the normed output times this weight
};

__device__ __forceinline__ float channel_log_decay(const ScanArgs& a, size_t row, int h, int i) {
  const float z = a.chan_a[row * a.ldca + (size_t)h * a.N + i];
  return a.chan_logit ? -a.chan_mult * softplus_f(-z) : z;
}

// One block a (head, request); the state in LDS as S[i * P + p], thread (part, p) walks its share
// of the keys i for value column p.  Tokens in turn: the recurrence as written.
template <typename T>
__global__ __launch_bounds__(256) void state_scan_kernel(ScanArgs a) {
  extern __shared__ float lds[];
  __shared__ float red[32];
  const int N = a.N, P = a.P, tid = threadIdx.x;
  const int h = blockIdx.x, r = blockIdx.y, hk = h / (a.H / a.Hk);
  const int parts = min(256 / P, N), chunk = (N + parts - 1) / parts;
  float* S = lds;
  float* qs = S + (size_t)N * P;
  float* ks = qs + N;
  float* vs = ks + N;
  float* partial = vs + P;  // [parts, P]
  float* as = partial + (size_t)parts * P;  // [N], where every key channel has a decay of its own
  const int start = a.seq_start[r], n = a.seq_len[r];
  float* Sg = a.state + (size_t)a.slot_ids[r] * a.state_stride + a.state_offset + (size_t)h * N * P;
  for (int base = 0; base < N * P; base += 256 * 8) {  // (eight loads a thread on their way at once)
    float sv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) sv[u] = Sg[min(base + u * 256 + tid, N * P - 1)];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (base + u * 256 + tid < N * P) S[base + u * 256 + tid] = sv[u];
  }
  const int half = a.rot_dims / 2;
  const int p = tid % P, part = tid / P;
  const bool works = tid < parts * P;
  const int i0 = part * chunk, i1 = min(N, i0 + chunk);
  for (int t = 0; t < n; ++t) {
    const size_t row = (size_t)(start + t);
    __syncthreads();  // the token before is done with qs, ks, vs, partial (and S is loaded)
    const float ksc = a.k_mult * (a.k_scale ? a.k_scale[row * a.H + h] : 1.0f);
    for (int i = tid; i < N; i += 256) {
      const float* qr = a.q + row * a.ldq + (size_t)hk * N;
      const float* kr = a.k + row * a.ldk + (size_t)hk * N;
      float qv = qr[i], kv = kr[i];
      if (i < a.rot_dims) {
        const int j = i < half ? i : i - half;
        float sn, cs;
        sincosf((float)a.positions[row] * a.inv_freq[j], &sn, &cs);
        if (i < half)
          qv = qr[j] * cs - qr[j + half] * sn, kv = kr[j] * cs - kr[j + half] * sn;
        else
          qv = qr[j + half] * cs + qr[j] * sn, kv = kr[j + half] * cs + kr[j] * sn;
      }
      qs[i] = qv, ks[i] = kv * ksc;
      if (a.chan_a) as[i] = expf(channel_log_decay(a, row, h, i));
    }
    for (int c = tid; c < P; c += 256) vs[c] = a.v[row * a.ldv + (size_t)h * P + c];
    const float at = a.chan_a ? 1.f : a.log_a ? expf(a.log_a[row * a.H + h]) : a.decay[h];
    __syncthreads();
    if (works) {
      const float vp = vs[p];
      float acc = 0.f;
      for (int i = i0; i < i1; ++i) {
        const float s = (a.chan_a ? as[i] : at) * S[(size_t)i * P + p] + ks[i] * vp;
        S[(size_t)i * P + p] = s;
        acc += s * qs[i];
      }
      partial[part * P + p] = acc;
    }
    __syncthreads();
    float o = 0.f;
    if (tid < P) {
      for (int j = 0; j < parts; ++j) o += partial[j * P + tid];
      if (a.skip) o += a.skip[h] * vs[tid];
    }
    if (a.unit_rms) {
      const float ss = block_sum(tid < P ? o * o : 0.f, red);
      o *= 1.0f / sqrtf(ss / (float)P + a.eps);
      if (a.norm_w && tid < P) o *= a.norm_w[tid];
    }
    if (tid < P) {
      if (a.gate) o *= silu_f(a.gate[row * a.ldg + (size_t)h * P + tid]);
      ((T*)a.out)[row * a.ldo + (size_t)h * P + tid] = from_f32<T>(o);
    }
  }
  __syncthreads();
  for (int i = tid; i < N * P; i += 256) Sg[i] = S[i];
}

// The same recurrence a chunk of C tokens at a time, for portions of many tokens: with
// L_t = log a_1 + ... + log a_t inside the chunk,
//   o_t = exp(L_t) S_0^T q_t + sum_(j <= t) exp(L_t - L_j) (q_t . k_j) v_j
//   S_C = exp(L_C) S_0 + sum_j exp(L_C - L_j) k_j v_j^T
// so a chunk is four small matrix products (q k^T, that times v, q S_0, k^T v) whose sums run over
// tokens side by side instead of one token after the other; every exponent is <= 0.  All in LDS,
// 32-bit, on the matrix cores (v_mfma_f32_16x16x4_f32, a wave a tile of 16 x 16): QT, KT
// [Np][C + 4] (transposed: a wave's operand is sixteen consecutive tokens), KW [C][Np] (keys times
// their decay to the chunk's end), V, O [C][Pp], AT [C][C + 4], S [Np][Pp]; Np, Pp: the head sizes
// rounded up to sixteen, the padding zero.
//
// Long portions are cut into spans of `span` tokens that run side by side (SpanArgs.mode): first
// every span's own contribution to the state, from zero, and its decay (SPAN_STATES); then, a
// thread an element, the state ahead of every span and the request's new state (span_states_kernel);
// then every span's outputs from the state ahead of it (SPAN_OUTPUTS).  WHOLE: a request's tokens
// in one block, chunk after chunk.
enum { WHOLE = 0, SPAN_STATES = 1, SPAN_OUTPUTS = 2 };
struct SpanArgs {
  int mode, span;
  const int* span_req;    // [spans] the request of a span
  const int* span_start;  // [spans] its first token, counted from the request's first of this step
  float* span_state;      // [spans, H, N * P]
  float* span_decay;      // [spans, H]
};

template <typename T>
__global__ __launch_bounds__(256) void state_chunks_kernel(ScanArgs a, int C, SpanArgs sp) {
  extern __shared__ float lds[];
  __shared__ float Lc[64], Lraw[64], Ksc[64], Rs[64];
  const int N = a.N, P = a.P, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int Np = (N + 15) & ~15, Pp = (P + 15) & ~15, CP = C + 4;
  const int h = blockIdx.x, hk = h / (a.H / a.Hk);
  const int r = sp.mode == WHOLE ? blockIdx.y : sp.span_req[blockIdx.y];
  float* QT = lds;
  float* KT = QT + (size_t)Np * CP;
  float* KW = KT + (size_t)Np * CP;
  float* V = KW + (size_t)C * Np;
  float* O = V + (size_t)C * Pp;
  float* AT = O + (size_t)C * Pp;
  float* S = AT + (size_t)C * CP;
  const int start = a.seq_start[r];
  const int lo = sp.mode == WHOLE ? 0 : sp.span_start[blockIdx.y];
  const int n = sp.mode == WHOLE ? a.seq_len[r] : min(a.seq_len[r], lo + sp.span);
  float* Sg = sp.mode == WHOLE ? a.state + (size_t)a.slot_ids[r] * a.state_stride + a.state_offset + (size_t)h * N * P
                               : sp.span_state + ((size_t)blockIdx.y * a.H + h) * N * P;
  for (int base = 0; base < Np * Pp; base += 256 * 8) {  // (eight loads a thread on their way at once)
    float sv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = min(base + u * 256 + tid, Np * Pp - 1), kn = min(i / Pp, N - 1), p = min(i % Pp, P - 1);
      sv[u] = sp.mode != SPAN_STATES ? Sg[(size_t)kn * P + p] : 0.f;  // (the same for every thread: no lane waits for another's load)
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = base + u * 256 + tid;
      if (i < Np * Pp) S[i] = i / Pp < N && i % Pp < P ? sv[u] : 0.f;
    }
  }
  const float log_decay = a.log_a ? 0.f : logf(a.decay[h]);
  const bool outputs = sp.mode != SPAN_STATES;
  float span_log = 0.f;
  for (int c0 = lo; c0 < n; c0 += C) {
    const int m = min(C, n - c0);
    const size_t row0 = (size_t)(start + c0);
    // Everything the chunk reads from memory is asked for at once, ahead of the barrier: a token's
    // decay and key scale (thread t < C), queries, keys (turned already, see the launcher) and
    // values sixteen a thread, and the gates that the rows meet on their way out.  Addresses are
    // pulled inside the chunk; what lies outside is zeroed when it is stored.  (Trips to memory one
    // after the other, not the products, are what a chunk's time is made of.)
    float lraw = 0.f, ksc = 1.f;
    if (tid < C) {
      const size_t rt = (row0 + min(tid, m - 1)) * a.H + h;
      lraw = tid < m ? (a.log_a ? a.log_a[rt] : log_decay) : 0.f;
      ksc = a.k_mult * (a.k_scale ? a.k_scale[rt] : 1.0f);
    }
    const bool gates_ahead = outputs && a.gate && P <= 64;
    float gv[16];
#pragma unroll
    for (int u = 0; u < 16; ++u)
      gv[u] = gates_ahead ? a.gate[(row0 + min(wave + 4 * u, m - 1)) * a.ldg + (size_t)h * P + min(lane, P - 1)] : 0.f;
    {
      const int total = C * N, v_total = C * P, most = max(total, v_total);
      const float* qb = a.q + row0 * a.ldq + (size_t)hk * N;
      const float* kb = a.k + row0 * a.ldk + (size_t)hk * N;
      const float* vb = a.v + row0 * a.ldv + (size_t)h * P;
      bool first = true;
      for (int base = 0; base < most; base += 256 * 16) {
        float qv[16], kv[16], vv[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int e = base + u * 256 + tid;
          const int eq = min(e, total - 1), t = eq / N, i = eq - t * N, tc = min(t, m - 1);
          qv[u] = qb[(size_t)tc * a.ldq + i], kv[u] = kb[(size_t)tc * a.ldk + i];
          const int ev = min(e, v_total - 1), tv = ev / P;
          vv[u] = vb[(size_t)min(tv, m - 1) * a.ldv + (ev - tv * P)];
        }
        if (first) __syncthreads();  // the chunk before is done with every array (and S is loaded)
        first = false;
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int e = base + u * 256 + tid;
          if (e < total) {
            const int t = e / N, i = e - t * N;
            QT[(size_t)i * CP + t] = t < m ? qv[u] : 0.f, KT[(size_t)i * CP + t] = t < m ? kv[u] : 0.f;
          }
          if (e < v_total) {
            const int t = e / P;
            V[(size_t)t * Pp + (e - t * P)] = t < m ? vv[u] : 0.f;
          }
        }
      }
      if (tid < C) Lraw[tid] = lraw, Ksc[tid] = ksc;
      for (int e = tid; e < C * (Np - N); e += 256) {  // the padding
        const int t = e / (Np - N), i = N + e % (Np - N);
        QT[(size_t)i * CP + t] = 0.f, KT[(size_t)i * CP + t] = 0.f;
      }
      for (int e = tid; e < C * (Pp - P); e += 256) V[(size_t)(e / (Pp - P)) * Pp + P + e % (Pp - P)] = 0.f;
    }
    __syncthreads();
    if (tid < C) {
      float acc = 0.f;  // (each of C threads adds its own prefix: C is at most 64)
      for (int t = 0; t <= tid; ++t) acc += Lraw[t];
      Lc[tid] = acc;
    }
    __syncthreads();
    const float L_end = Lc[m - 1];
    for (int e = tid; e < C * Np; e += 256) {
      const int j = e / Np, i = e % Np;
      KW[e] = j < m ? KT[(size_t)i * CP + j] * (Ksc[j] * expf(L_end - Lc[j])) : 0.f;
    }
    span_log += L_end;
    // The three products run on the matrix cores in 32-bit (v_mfma_f32_16x16x4_f32: lane l brings
    // A[l % 16][l / 16] and B[l / 16][l % 16] and gets D[4 (l / 16) + x][l % 16]); a wave a tile
    // of 16 x 16.  AT[j][t] = (q_t . k_j) exp(L_t - L_j) for j <= t, else 0
    const int ct = C / 16, lr = lane & 15, lg = lane >> 4;
    for (int tile = wave; outputs && tile < ct * ct; tile += 4) {
      const int t0 = (tile / ct) * 16, j0 = (tile % ct) * 16;
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
      if (j0 <= t0 + 15)
        for (int i = 0; i < Np; i += 4)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(QT[(size_t)(i + lg) * CP + t0 + lr], KT[(size_t)(i + lg) * CP + j0 + lr], acc, 0, 0, 0);
      // D[m = t][n = j]: this lane holds t = t0 + 4 lg + x for j = j0 + lr
      const int j = j0 + lr;
      float4 o;
      float* ov = &o.x;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int t = t0 + 4 * lg + x;
        ov[x] = j <= t && t < m ? acc[x] * (Ksc[j] * expf(Lc[t] - Lc[j])) : 0.f;
      }
      *(float4*)(AT + (size_t)j * CP + t0 + 4 * lg) = o;
    }
    __syncthreads();
    // O[t][p] = sum_j AT[j][t] V[j][p] + exp(L_t) sum_i QT[i][t] S[i][p]  (+ skip v)
    const int pt = Pp / 16;
    for (int tile = wave; outputs && tile < ct * pt; tile += 4) {
      const int t0 = (tile / pt) * 16, p0 = (tile % pt) * 16;
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f}, old = {0.f, 0.f, 0.f, 0.f};
      const int j_end = min((m + 3) & ~3, t0 + 16);  // (AT is zero where j > t or t >= m, V where j >= m)
      for (int j = 0; j < j_end; j += 4)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(AT[(size_t)(j + lg) * CP + t0 + lr], V[(size_t)(j + lg) * Pp + p0 + lr], acc, 0, 0, 0);
      for (int i = 0; i < Np; i += 4)
        old = __builtin_amdgcn_mfma_f32_16x16x4f32(QT[(size_t)(i + lg) * CP + t0 + lr], S[(size_t)(i + lg) * Pp + p0 + lr], old, 0, 0, 0);
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int t = t0 + 4 * lg + x, pcol = p0 + lr;
        float o = acc[x] + expf(Lc[min(t, m - 1)]) * old[x];
        if (a.skip) o += a.skip[h] * V[(size_t)t * Pp + pcol];
        O[(size_t)t * Pp + pcol] = o;
      }
    }
    __syncthreads();
    // S = exp(L_end) S + KW^T V
    const float shrink = expf(L_end);
    const int nt = Np / 16;
    const bool state_needed = sp.mode != SPAN_OUTPUTS || c0 + C < n;  // (a span's outputs: nobody reads the state after its last chunk)
    for (int tile = wave; state_needed && tile < nt * pt; tile += 4) {
      const int i0 = (tile / pt) * 16, p0 = (tile % pt) * 16;
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
      const int j_end = (m + 3) & ~3;  // (KW and V are zero from m on)
      for (int j = 0; j < j_end; j += 4)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(KW[(size_t)(j + lg) * Np + i0 + lr], V[(size_t)(j + lg) * Pp + p0 + lr], acc, 0, 0, 0);
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        float* sp_ = S + (size_t)(i0 + 4 * lg + x) * Pp + p0 + lr;
        *sp_ = shrink * *sp_ + acc[x];
      }
    }
    // the rows on their way out: a wave a token; the gates of eight tokens are asked for at once
    if (outputs && a.unit_rms)
      for (int t = wave; t < m; t += 4) {
        float ss = 0.f;
        for (int pc = lane; pc < P; pc += 64) ss += O[(size_t)t * Pp + pc] * O[(size_t)t * Pp + pc];
        ss = wave_sum(ss);
        if (lane == 0) Rs[t] = 1.0f / sqrtf(ss / (float)P + a.eps);
      }
    // (a wave reads the Rs it wrote itself: tokens wave, wave + 4, ...)
    if (gates_ahead || (outputs && !a.gate && P <= 64)) {
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int t = wave + 4 * u;
        if (t >= m || lane >= P) continue;
        float o = O[(size_t)t * Pp + lane];
        if (a.unit_rms) o *= Rs[t];
        if (a.gate) o *= silu_f(gv[u]);
        ((T*)a.out)[(row0 + t) * a.ldo + (size_t)h * P + lane] = from_f32<T>(o);
      }
    } else {
      for (int pb = 0; outputs && pb < P; pb += 64) {
        const int pc = min(pb + lane, P - 1);
        for (int tb = wave; tb < m; tb += 32) {
          float g8[8];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            g8[u] = a.gate ? a.gate[(row0 + min(tb + 4 * u, m - 1)) * a.ldg + (size_t)h * P + pc] : 0.f;
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int t = tb + 4 * u;
            if (t >= m || pb + lane >= P) continue;
            float o = O[(size_t)t * Pp + pc];
            if (a.unit_rms) o *= Rs[t];
            if (a.gate) o *= silu_f(g8[u]);
            ((T*)a.out)[(row0 + t) * a.ldo + (size_t)h * P + pc] = from_f32<T>(o);
          }
        }
      }
    }
  }
  __syncthreads();
  if (sp.mode == SPAN_OUTPUTS) return;
  for (int i = tid; i < N * P; i += 256) Sg[i] = S[(size_t)(i / P) * Pp + i % P];
  if (sp.mode == SPAN_STATES && tid == 0) sp.span_decay[(size_t)blockIdx.y * a.H + h] = expf(span_log);
}

// The same chunks where every key channel i has a decay of its own (a.chan_a): with L_t[i] the sum
// of the channel's log decays inside the chunk,
//   o_t  = sum_i q_t[i] exp(L_t[i]) S_0[i, :] + sum_(j <= t) A[t][j] v_j,
//   A[t][j] = sum_i q_t[i] k_j[i] exp(L_t[i] - L_j[i]),
//   S_C[i, :] = exp(L_C[i]) S_0[i, :] + sum_j k_j[i] exp(L_C[i] - L_j[i]) v_j
// A does not split into a product of a factor of t and a factor of j whose exponents both stay
// <= 0, so it is made tile by tile (16 x 16 tokens): below the diagonal both operands are taken
// to the reference b = the last token ahead of the tile's queries, q_t exp(L_t - L_b) and
// k_j exp(L_b - L_j) (j <= b < t: both exponents <= 0), on the matrix cores; on the diagonal every
// pair (t, j <= t) is summed as written, four lanes a pair, each a quarter of the channels, added
// in a fixed order.  LT [Np][C + 4] holds L; afterwards QT becomes q exp(L_t) and KT becomes
// k exp(L_C - L_j) in place, for the products with the state and into it.
template <typename T>
__global__ __launch_bounds__(256) void channel_chunks_kernel(ScanArgs a, int C, SpanArgs sp) {
  extern __shared__ float lds[];
  __shared__ float Rs[64];
  __shared__ unsigned char pair_t[136], pair_j[136];
  const int N = a.N, P = a.P, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int Np = (N + 15) & ~15, Pp = (P + 15) & ~15, CP = C + 4;
  const int h = blockIdx.x;
  const int r = sp.mode == WHOLE ? blockIdx.y : sp.span_req[blockIdx.y];
  float* QT = lds;
  float* KT = QT + (size_t)Np * CP;
  float* LT = KT + (size_t)Np * CP;
  float* V = LT + (size_t)Np * CP;
  float* O = V + (size_t)C * Pp;
  float* AT = O + (size_t)C * Pp;
  float* S = AT + (size_t)C * CP;
  float* Lsum = S + (size_t)Np * Pp;  // [Np] the log decay of every channel over the span so far
  const int start = a.seq_start[r];
  const int lo = sp.mode == WHOLE ? 0 : sp.span_start[blockIdx.y];
  const int n = sp.mode == WHOLE ? a.seq_len[r] : min(a.seq_len[r], lo + sp.span);
  float* Sg = sp.mode == WHOLE ? a.state + (size_t)a.slot_ids[r] * a.state_stride + a.state_offset + (size_t)h * N * P
                               : sp.span_state + ((size_t)blockIdx.y * a.H + h) * N * P;
  for (int base = 0; base < Np * Pp; base += 256 * 8) {
    float sv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = min(base + u * 256 + tid, Np * Pp - 1), kn = min(i / Pp, N - 1), p = min(i % Pp, P - 1);
      sv[u] = sp.mode != SPAN_STATES ? Sg[(size_t)kn * P + p] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = base + u * 256 + tid;
      if (i < Np * Pp) S[i] = i / Pp < N && i % Pp < P ? sv[u] : 0.f;
    }
  }
  for (int i = tid; i < Np; i += 256) Lsum[i] = 0.f;
  if (tid < 136) {  // the pairs (t, j <= t) of a tile of sixteen tokens, row by row
    int t = 0;
    while ((t + 1) * (t + 2) / 2 <= tid) ++t;
    pair_t[tid] = (unsigned char)t, pair_j[tid] = (unsigned char)(tid - t * (t + 1) / 2);
  }
  const bool outputs = sp.mode != SPAN_STATES;
  const int ct = C / 16, pt = Pp / 16, nt = Np / 16, lr = lane & 15, lg = lane >> 4;
  for (int c0 = lo; c0 < n; c0 += C) {
    const int m = min(C, n - c0);
    const size_t row0 = (size_t)(start + c0);
    const bool gates_ahead = outputs && a.gate && P <= 64;
    float gv[16];
#pragma unroll
    for (int u = 0; u < 16; ++u)
      gv[u] = gates_ahead ? a.gate[(row0 + min(wave + 4 * u, m - 1)) * a.ldg + (size_t)h * P + min(lane, P - 1)] : 0.f;
    {
      const int total = C * N, v_total = C * P, most = max(total, v_total);
      const float* qb = a.q + row0 * a.ldq + (size_t)h * N;
      const float* kb = a.k + row0 * a.ldk + (size_t)h * N;
      const float* ab = a.chan_a + row0 * a.ldca + (size_t)h * N;
      const float* vb = a.v + row0 * a.ldv + (size_t)h * P;
      bool first = true;
      for (int base = 0; base < most; base += 256 * 16) {
        float qv[16], kv[16], av[16], vv[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int e = base + u * 256 + tid;
          const int eq = min(e, total - 1), t = eq / N, i = eq - t * N, tc = min(t, m - 1);
          qv[u] = qb[(size_t)tc * a.ldq + i], kv[u] = kb[(size_t)tc * a.ldk + i], av[u] = ab[(size_t)tc * a.ldca + i];
          const int ev = min(e, v_total - 1), tv = ev / P;
          vv[u] = vb[(size_t)min(tv, m - 1) * a.ldv + (ev - tv * P)];
        }
        if (first) {
          __syncthreads();  // the chunk before is done with every array (and S is loaded)
          for (int e = tid; e < C * CP; e += 256) AT[e] = 0.f;
        }
        first = false;
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int e = base + u * 256 + tid;
          if (e < total) {
            const int t = e / N, i = e - t * N;
            const float la = a.chan_logit ? -a.chan_mult * softplus_f(-av[u]) : av[u];
            QT[(size_t)i * CP + t] = t < m ? qv[u] : 0.f, KT[(size_t)i * CP + t] = t < m ? kv[u] * a.k_mult : 0.f;
            LT[(size_t)i * CP + t] = t < m ? la : 0.f;
          }
          if (e < v_total) {
            const int t = e / P;
            V[(size_t)t * Pp + (e - t * P)] = t < m ? vv[u] : 0.f;
          }
        }
      }
      for (int e = tid; e < C * (Np - N); e += 256) {  // the padding
        const int t = e / (Np - N), i = N + e % (Np - N);
        QT[(size_t)i * CP + t] = 0.f, KT[(size_t)i * CP + t] = 0.f, LT[(size_t)i * CP + t] = 0.f;
      }
      for (int e = tid; e < C * (Pp - P); e += 256) V[(size_t)(e / (Pp - P)) * Pp + P + e % (Pp - P)] = 0.f;
    }
    __syncthreads();
    for (int i = tid; i < N; i += 256) {  // a channel's running sum, token after token
      float acc = 0.f;
      for (int t = 0; t < C; ++t) {
        acc += LT[(size_t)i * CP + t];
        LT[(size_t)i * CP + t] = acc;
      }
      Lsum[i] += acc;
    }
    __syncthreads();
    if (outputs) {
      // the diagonal tiles: lanes 4p .. 4p + 3 share pair p, a quarter of the channels each
      const int items = ct * 136 * 4, quarter = Np / 4, part = tid & 3;
      for (int base = 0; base < items; base += 256) {
        const int item = base + tid, pr = min(item, items - 1) >> 2, tile = pr / 136, pp = pr - tile * 136;
        const int t = tile * 16 + pair_t[pp], j = tile * 16 + pair_j[pp];
        float acc = 0.f;
        for (int i = part * quarter; i < (part + 1) * quarter; ++i) {
          const float* row = QT + (size_t)i * CP;
          const float* lrow = LT + (size_t)i * CP;
          acc += row[t] * KT[(size_t)i * CP + j] * expf(lrow[t] - lrow[j]);
        }
        acc += __shfl_xor(acc, 1);
        acc += __shfl_xor(acc, 2);
        if (item < items && part == 0) AT[(size_t)j * CP + t] = acc;
      }
      // the tiles below the diagonal
      const int below = ct * (ct - 1) / 2;
      for (int tile = wave; tile < below; tile += 4) {
        int tt = 1;
        while (tt * (tt + 1) / 2 <= tile) ++tt;
        const int t0 = tt * 16, j0 = (tile - tt * (tt - 1) / 2) * 16;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        for (int i = 0; i < Np; i += 4) {
          const size_t ro = (size_t)(i + lg) * CP;
          const float ref = LT[ro + t0 - 1];
          const float qa = QT[ro + t0 + lr] * expf(LT[ro + t0 + lr] - ref);
          const float kb_ = KT[ro + j0 + lr] * expf(ref - LT[ro + j0 + lr]);
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(qa, kb_, acc, 0, 0, 0);
        }
        float4 o = {acc[0], acc[1], acc[2], acc[3]};
        *(float4*)(AT + (size_t)(j0 + lr) * CP + t0 + 4 * lg) = o;
      }
    }
    __syncthreads();
    const bool state_needed = sp.mode != SPAN_OUTPUTS || c0 + C < n;
    for (int e = tid; e < Np * C; e += 256) {
      const int i = e / C, t = e - i * C;
      const size_t at = (size_t)i * CP + t;
      const float l = LT[at];
      if (outputs) QT[at] *= expf(l);
      if (state_needed) KT[at] *= expf(LT[(size_t)i * CP + C - 1] - l);  // (from m on the sum stands still: L_C)
    }
    __syncthreads();
    // O[t][p] = sum_j AT[j][t] V[j][p] + sum_i QT[i][t] S[i][p]
    for (int tile = wave; outputs && tile < ct * pt; tile += 4) {
      const int t0 = (tile / pt) * 16, p0 = (tile % pt) * 16;
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
      const int j_end = min((m + 3) & ~3, t0 + 16);
      for (int j = 0; j < j_end; j += 4)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(AT[(size_t)(j + lg) * CP + t0 + lr], V[(size_t)(j + lg) * Pp + p0 + lr], acc, 0, 0, 0);
      for (int i = 0; i < Np; i += 4)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(QT[(size_t)(i + lg) * CP + t0 + lr], S[(size_t)(i + lg) * Pp + p0 + lr], acc, 0, 0, 0);
#pragma unroll
      for (int x = 0; x < 4; ++x) O[(size_t)(t0 + 4 * lg + x) * Pp + p0 + lr] = acc[x];
    }
    __syncthreads();
    // S[i][:] = exp(L_C[i]) S[i][:] + sum_j KT[i][j] V[j][:]
    for (int tile = wave; state_needed && tile < nt * pt; tile += 4) {
      const int i0 = (tile / pt) * 16, p0 = (tile % pt) * 16;
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
      const int j_end = (m + 3) & ~3;
      for (int j = 0; j < j_end; j += 4)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(KT[(size_t)(i0 + lr) * CP + j + lg], V[(size_t)(j + lg) * Pp + p0 + lr], acc, 0, 0, 0);
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int i = i0 + 4 * lg + x;
        float* sp_ = S + (size_t)i * Pp + p0 + lr;
        *sp_ = expf(LT[(size_t)i * CP + C - 1]) * *sp_ + acc[x];
      }
    }
    // the rows on their way out: a wave a token
    if (outputs && a.unit_rms)
      for (int t = wave; t < m; t += 4) {
        float ss = 0.f;
        for (int pc = lane; pc < P; pc += 64) ss += O[(size_t)t * Pp + pc] * O[(size_t)t * Pp + pc];
        ss = wave_sum(ss);
        if (lane == 0) Rs[t] = 1.0f / sqrtf(ss / (float)P + a.eps);
      }
    if (gates_ahead || (outputs && !a.gate && P <= 64)) {
      const float nw = a.norm_w && a.unit_rms ? a.norm_w[min(lane, P - 1)] : 1.f;
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int t = wave + 4 * u;
        if (t >= m || lane >= P) continue;
        float o = O[(size_t)t * Pp + lane];
        if (a.unit_rms) o *= Rs[t] * nw;
        if (a.gate) o *= silu_f(gv[u]);
        ((T*)a.out)[(row0 + t) * a.ldo + (size_t)h * P + lane] = from_f32<T>(o);
      }
    } else {
      for (int pb = 0; outputs && pb < P; pb += 64) {
        const int pc = min(pb + lane, P - 1);
        const float nw = a.norm_w && a.unit_rms ? a.norm_w[pc] : 1.f;
        for (int tb = wave; tb < m; tb += 32) {
          float g8[8];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            g8[u] = a.gate ? a.gate[(row0 + min(tb + 4 * u, m - 1)) * a.ldg + (size_t)h * P + pc] : 0.f;
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int t = tb + 4 * u;
            if (t >= m || pb + lane >= P) continue;
            float o = O[(size_t)t * Pp + pc];
            if (a.unit_rms) o *= Rs[t] * nw;
            if (a.gate) o *= silu_f(g8[u]);
            ((T*)a.out)[(row0 + t) * a.ldo + (size_t)h * P + pc] = from_f32<T>(o);
          }
        }
      }
    }
  }
  __syncthreads();
  if (sp.mode == SPAN_OUTPUTS) return;
  for (int i = tid; i < N * P; i += 256) Sg[i] = S[(size_t)(i / P) * Pp + i % P];
  if (sp.mode == SPAN_STATES)  // (span_decay has a value for every channel here)
    for (int i = tid; i < N; i += 256) sp.span_decay[((size_t)blockIdx.y * a.H + h) * N + i] = expf(Lsum[i]);
}

// Block (head, request, 256 elements of the state), a thread an element: span_state[s] becomes
// the state ahead of span s, and the request's row its state after the last span.  Four spans'
// values are asked for before the first is used.  With decays per key channel span_decay is
// [spans, H, N], else [spans, H].
__global__ __launch_bounds__(256) void span_states_kernel(ScanArgs a, SpanArgs sp, const int* __restrict__ span_first) {
  const int h = blockIdx.x, r = blockIdx.y, NP = a.N * a.P, i = blockIdx.z * 256 + threadIdx.x;
  if (i >= NP) return;
  const int first = span_first[r], n_spans = (a.seq_len[r] + sp.span - 1) / sp.span;
  float* Sg = a.state + (size_t)a.slot_ids[r] * a.state_stride + a.state_offset + (size_t)h * NP;
  float s = Sg[i];
  for (int c0 = 0; c0 < n_spans; c0 += 4) {
    float add[4], dec[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = min(c0 + u, n_spans - 1);
      add[u] = sp.span_state[((size_t)(first + c) * a.H + h) * NP + i];
      dec[u] = a.chan_a ? sp.span_decay[((size_t)(first + c) * a.H + h) * a.N + i / a.P] : sp.span_decay[(size_t)(first + c) * a.H + h];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (c0 + u >= n_spans) break;
      sp.span_state[((size_t)(first + c0 + u) * a.H + h) * NP + i] = s;
      s = dec[u] * s + add[u];
    }
  }
  Sg[i] = s;
}

// Queries and keys turned in place ahead of the kernels that take chunks (which would otherwise
// each turn them again): thread (token, key head, pair of columns).
__global__ __launch_bounds__(256) void rotate_pairs_kernel(float* __restrict__ q, int ldq, float* __restrict__ k, int ldk,
                                                           const int* __restrict__ positions,
                                                           const float* __restrict__ inv_freq, int n_tokens, int heads,
                                                           int N, int half) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long)n_tokens * heads * half) return;
  const int j = e % half, hd = (e / half) % heads;
  const long t = e / ((long)half * heads);
  float sn, cs;
  sincosf((float)positions[t] * inv_freq[j], &sn, &cs);
  float* qr = q + t * ldq + (size_t)hd * N;
  float* kr = k + t * ldk + (size_t)hd * N;
  const float qa = qr[j], qb = qr[j + half], ka = kr[j], kb = kr[j + half];
  qr[j] = qa * cs - qb * sn, qr[j + half] = qb * cs + qa * sn;
  kr[j] = ka * cs - kb * sn, kr[j + half] = kb * cs + ka * sn;
}

// ---------------------------------------------------------------------------

// Thread (token row, channel c): c < C is a convolution channel, C <= c < C + H a head's step size.
__global__ __launch_bounds__(256) void ssm_prepare_kernel(
    const float* __restrict__ u, int ldu, int conv_col, int dt_col, const float* __restrict__ w,
    const float* __restrict__ b, int taps, int C, int H, const float* __restrict__ dt_bias,
    const float* __restrict__ A_log, float* __restrict__ state, size_t state_stride, size_t conv_offset,
    const int* __restrict__ token_req, const int* __restrict__ seq_start, const int* __restrict__ slot_ids,
    float* __restrict__ xbc, float* __restrict__ dt, float* __restrict__ log_a, int n_tokens, int single_tokens) {
  const int c = blockIdx.y * 256 + threadIdx.x, row = blockIdx.x;
  if (c >= C + H) return;
  if (c >= C) {
    const int hd = c - C;
    const float d = softplus_f(u[(size_t)row * ldu + dt_col + hd] + dt_bias[hd]);
    dt[(size_t)row * H + hd] = d;
    log_a[(size_t)row * H + hd] = -expf(A_log[hd]) * d;
    return;
  }
  const int req = token_req[row], local = row - seq_start[req];
  float* old = state + (size_t)slot_ids[req] * state_stride + conv_offset;  // [taps - 1, C], the latest last
  float acc = b ? b[c] : 0.f;
  for (int j = taps - 1; j >= 0; --j) {  // the oldest input first
    const int at = local - j;
    const float in = at >= 0 ? u[(size_t)(row - j) * ldu + conv_col + c] : old[(size_t)(taps - 1 + at) * C + c];
    acc += w[(size_t)c * taps + (taps - 1 - j)] * in;
    // every request brings one token: this thread is the only one that reads or writes its
    // request's inputs of channel c, so it moves them up by one as it goes (the oldest first)
    if (single_tokens && j < taps - 1) old[(size_t)(taps - 2 - j) * C + c] = in;
  }
  xbc[(size_t)row * C + c] = silu_f(acc);
}

// Thread (request, channel): the new last taps - 1 inputs, ascending, so that what is still to be
// read of the old ones lies ahead of what is written.
__global__ __launch_bounds__(256) void conv_state_update_kernel(const float* __restrict__ u, int ldu, int conv_col,
                                                                int taps, int C, float* __restrict__ state,
                                                                size_t state_stride, size_t conv_offset,
                                                                const int* __restrict__ seq_start,
                                                                const int* __restrict__ seq_len,
                                                                const int* __restrict__ slot_ids) {
  const int c = blockIdx.x * 256 + threadIdx.x, req = blockIdx.y;
  if (c >= C) return;
  const int start = seq_start[req], n = seq_len[req];
  float* st = state + (size_t)slot_ids[req] * state_stride + conv_offset;
  for (int j = 0; j < taps - 1; ++j) {
    const int at = n - (taps - 1) + j;
    st[(size_t)j * C + c] = at >= 0 ? u[(size_t)(start + at) * ldu + conv_col + c] : st[(size_t)(j + n) * C + c];
  }
}

// A block a (row, group).
template <typename T>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_kernel(const float* __restrict__ y, int ldy,
                                                                  const float* __restrict__ z, int ldz,
                                                                  const float* __restrict__ w, float eps, int size,
                                                                  T* __restrict__ out, int ldo) {
  __shared__ float red[32];
  const int row = blockIdx.x, g = blockIdx.y, tid = threadIdx.x;
  const float* yr = y + (size_t)row * ldy + (size_t)g * size;
  const float* zr = z + (size_t)row * ldz + (size_t)g * size;
  float q = 0.f;
  for (int k = tid; k < size; k += 256) {
    const float s = yr[k] * silu_f(zr[k]);
    q += s * s;
  }
  const float rstd = 1.0f / sqrtf(block_sum(q, red) / (float)size + eps);
  for (int k = tid; k < size; k += 256)
    out[(size_t)row * ldo + (size_t)g * size + k] = from_f32<T>(yr[k] * silu_f(zr[k]) * rstd * w[(size_t)g * size + k]);
}

DEFINE_LAST_ERROR(mlxlm_last_error)

#define SCAN_MAX_LDS (158 * 1024)

// Floats of LDS that the chunked kernel needs for chunks of C tokens.
static size_t chunk_floats(int N, int P, int C) {
  const size_t Np = (N + 15) & ~15, Pp = (P + 15) & ~15, CP = C + 4;
  return 2 * Np * CP + (size_t)C * Np + 2 * (size_t)C * Pp + (size_t)C * CP + Np * Pp;
}
// The same for the kernel with a decay per key channel.
static size_t channel_chunk_floats(int N, int P, int C) {
  const size_t Np = (N + 15) & ~15, Pp = (P + 15) & ~15, CP = C + 4;
  return 3 * Np * CP + 2 * (size_t)C * Pp + (size_t)C * CP + Np * Pp + Np;
}

// `chunked`: the kernel that takes a chunk of tokens at a time (for steps in which some request
// brings many tokens); otherwise, or where not even chunks of 16 fit the LDS, token by token.
// `chunked`: 0 token by token; 1 chunks of tokens, a request a block; 2 chunks, the requests cut
// into spans of `span` tokens that run side by side (n_spans of them: span_req, span_start; the
// first span of every request in span_first; span_state: room for n_spans * H * N * P floats,
// span_decay: for n_spans * H, with a decay per key channel for n_spans * H * N).
extern "C" int state_scan(const ScanArgs* args, int chunked, int span, int n_spans, const int* span_req,
                          const int* span_start, const int* span_first, float* span_state, float* span_decay,
                          hipStream_t stream) {
  const ScanArgs& a = *args;
  if (a.n_requests <= 0 || a.H <= 0) return 0;
  if (!a.q || !a.k || !a.v || !a.out || !a.state || !a.seq_start || !a.seq_len || !a.slot_ids)
    FAIL("state_scan: null pointer");
  if (a.N <= 0 || a.P <= 0 || a.P > 256) FAIL("state_scan: key size %d, value size %d (at most 256)", a.N, a.P);
  if (a.Hk <= 0 || a.H % a.Hk) FAIL("state_scan: %d heads over %d key heads", a.H, a.Hk);
  if (!a.log_a && !a.decay && !a.chan_a) FAIL("state_scan: a decay per token, per head or per key channel is needed");
  if (a.chan_a && (a.ldca < a.H * a.N || a.Hk != a.H)) FAIL("state_scan: decays per key channel come in rows of heads x keys");
  if (a.rot_dims && (a.rot_dims % 2 || a.rot_dims > a.N || !a.inv_freq || !a.positions))
    FAIL("state_scan: %d turning columns of %d", a.rot_dims, a.N);
  if (a.ldq < a.Hk * a.N || a.ldk < a.Hk * a.N || a.ldv < a.H * a.P || a.ldo < a.H * a.P || (a.gate && a.ldg < a.H * a.P))
    FAIL("state_scan: a row is narrower than its heads");
  if (a.out_dtype != DT_F32 && a.out_dtype != DT_BF16) FAIL("state_scan: unknown dtype code %d", a.out_dtype);
  const int parts = a.N < 256 / a.P ? a.N : 256 / a.P;
  const size_t lds = ((size_t)a.N * a.P + 3 * (size_t)a.N + a.P + (size_t)parts * a.P) * sizeof(float);
  if (lds > SCAN_MAX_LDS) FAIL("state_scan: a state of %d x %d does not fit a block's LDS", a.N, a.P);
  static bool raised = false;
  if (!raised) {
    (void)hipFuncSetAttribute((const void*)state_scan_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, SCAN_MAX_LDS);
    (void)hipFuncSetAttribute((const void*)state_scan_kernel<bf16>, hipFuncAttributeMaxDynamicSharedMemorySize, SCAN_MAX_LDS);
    raised = true;
  }
  dim3 grid(a.H, a.n_requests), block(256);
  int C = 0;
  // (the chunks with a decay per key channel know neither a scale per token, a skip nor a rotation)
  const bool by_channel = a.chan_a != nullptr;
  if (chunked && !(by_channel && (a.k_scale || a.skip || a.rot_dims)))
    for (int c = 64; c >= 16 && !C; c /= 2)
      if ((by_channel ? channel_chunk_floats(a.N, a.P, c) : chunk_floats(a.N, a.P, c)) * sizeof(float) <= SCAN_MAX_LDS) C = c;
  if (C) {
    ScanArgs turned = a;  // (the chunked kernel itself turns nothing)
    if (a.rot_dims) {
      // (q and k are the caller's work memory: the projection's rows, which nothing reads after this)
      const long items = (long)a.n_tokens_hint * a.Hk * (a.rot_dims / 2);
      if (a.n_tokens_hint <= 0) FAIL("state_scan: the chunked kernels need the number of token rows");
      hipLaunchKernelGGL(rotate_pairs_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, (float*)a.q, a.ldq,
                         (float*)a.k, a.ldk, a.positions, a.inv_freq, a.n_tokens_hint, a.Hk, a.N, a.rot_dims / 2);
      turned.rot_dims = 0;
    }
    static bool chunks_raised = false;
    if (!chunks_raised) {
      (void)hipFuncSetAttribute((const void*)state_chunks_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, SCAN_MAX_LDS);
      (void)hipFuncSetAttribute((const void*)state_chunks_kernel<bf16>, hipFuncAttributeMaxDynamicSharedMemorySize, SCAN_MAX_LDS);
      (void)hipFuncSetAttribute((const void*)channel_chunks_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, SCAN_MAX_LDS);
      (void)hipFuncSetAttribute((const void*)channel_chunks_kernel<bf16>, hipFuncAttributeMaxDynamicSharedMemorySize, SCAN_MAX_LDS);
      chunks_raised = true;
    }
    const size_t bytes = (by_channel ? channel_chunk_floats(a.N, a.P, C) : chunk_floats(a.N, a.P, C)) * sizeof(float);
    SpanArgs sp = {WHOLE, 0, nullptr, nullptr, nullptr, nullptr};
#define CHUNKS(GRID)                                                                                \
  do {                                                                                              \
    if (by_channel && a.out_dtype == DT_F32)                                                        \
      hipLaunchKernelGGL(channel_chunks_kernel<float>, GRID, block, bytes, stream, turned, C, sp);       \
    else if (by_channel)                                                                            \
      hipLaunchKernelGGL(channel_chunks_kernel<bf16>, GRID, block, bytes, stream, turned, C, sp);        \
    else if (a.out_dtype == DT_F32)                                                                 \
      hipLaunchKernelGGL(state_chunks_kernel<float>, GRID, block, bytes, stream, turned, C, sp);         \
    else                                                                                            \
      hipLaunchKernelGGL(state_chunks_kernel<bf16>, GRID, block, bytes, stream, turned, C, sp);          \
  } while (0)
    if (chunked == 2 && n_spans > 0) {
      if (!span_req || !span_start || !span_first || !span_state || !span_decay) FAIL("state_scan: null pointer among the spans' arrays");
      if (span < C || span % C) FAIL("state_scan: spans of %d tokens in chunks of %d", span, C);
      dim3 span_grid(a.H, n_spans);
      sp = SpanArgs{SPAN_STATES, span, span_req, span_start, span_state, span_decay};
      CHUNKS(span_grid);
      hipLaunchKernelGGL(span_states_kernel, dim3(a.H, a.n_requests, (a.N * a.P + 255) / 256), block, 0, stream, turned, sp, span_first);
      sp.mode = SPAN_OUTPUTS;
      CHUNKS(span_grid);
    } else {
      CHUNKS(grid);
    }
#undef CHUNKS
    CHECK_LAUNCH("state_scan");
    return 0;
  }
  if (a.out_dtype == DT_F32)
    hipLaunchKernelGGL(state_scan_kernel<float>, grid, block, lds, stream, a);
  else
    hipLaunchKernelGGL(state_scan_kernel<bf16>, grid, block, lds, stream, a);
  CHECK_LAUNCH("state_scan");
  return 0;
}

// `single_tokens`: every request brings one token (the caller says so); the kernel then also moves
// the requests' last inputs up by one, and no conv_state_update follows.
extern "C" int ssm_prepare(const float* u, int ldu, int conv_col, int dt_col, const float* w, const float* b, int taps,
                           int C, int H, const float* dt_bias, const float* A_log, float* state,
                           size_t state_stride, size_t conv_offset, const int* token_req, const int* seq_start,
                           const int* slot_ids, float* xbc, float* dt, float* log_a, int n_tokens, int single_tokens,
                           hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (!u || !w || !dt_bias || !A_log || !state || !token_req || !seq_start || !slot_ids || !xbc || !dt || !log_a)
    FAIL("ssm_prepare: null pointer");
  if (taps < 1 || C <= 0 || H <= 0 || conv_col < 0 || dt_col < 0 || conv_col + C > ldu || dt_col + H > ldu)
    FAIL("ssm_prepare: %d taps, %d channels from column %d, %d heads from column %d, rows of %d", taps, C, conv_col, H, dt_col, ldu);
  dim3 grid(n_tokens, (C + H + 255) / 256), block(256);
  hipLaunchKernelGGL(ssm_prepare_kernel, grid, block, 0, stream, u, ldu, conv_col, dt_col, w, b, taps, C, H, dt_bias,
                     A_log, state, state_stride, conv_offset, token_req, seq_start, slot_ids, xbc, dt, log_a, n_tokens, single_tokens);
  CHECK_LAUNCH("ssm_prepare");
  return 0;
}

extern "C" int conv_state_update(const float* u, int ldu, int conv_col, int taps, int C, float* state,
                                 size_t state_stride, size_t conv_offset, const int* seq_start, const int* seq_len,
                                 const int* slot_ids, int n_requests, hipStream_t stream) {
  if (n_requests <= 0 || taps <= 1) return 0;
  if (!u || !state || !seq_start || !seq_len || !slot_ids) FAIL("conv_state_update: null pointer");
  if (C <= 0 || conv_col < 0 || conv_col + C > ldu) FAIL("conv_state_update: %d channels from column %d in rows of %d", C, conv_col, ldu);
  dim3 grid((C + 255) / 256, n_requests), block(256);
  hipLaunchKernelGGL(conv_state_update_kernel, grid, block, 0, stream, u, ldu, conv_col, taps, C, state, state_stride,
                     conv_offset, seq_start, seq_len, slot_ids);
  CHECK_LAUNCH("conv_state_update");
  return 0;
}

extern "C" int gated_group_rmsnorm(const float* y, int ldy, const float* z, int ldz, const float* w, float eps,
                                   int n_rows, int width, int groups, void* out, int ldo, int out_dtype,
                                   hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!y || !z || !w || !out) FAIL("gated_group_rmsnorm: null pointer");
  if (groups <= 0 || width <= 0 || width % groups || ldy < width || ldz < width || ldo < width)
    FAIL("gated_group_rmsnorm: width %d in %d groups, row strides %d, %d, %d", width, groups, ldy, ldz, ldo);
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) FAIL("gated_group_rmsnorm: unknown dtype code %d", out_dtype);
  dim3 grid(n_rows, groups), block(256);
  if (out_dtype == DT_F32)
    hipLaunchKernelGGL(gated_group_rmsnorm_kernel<float>, grid, block, 0, stream, y, ldy, z, ldz, w, eps, width / groups, (float*)out, ldo);
  else
    hipLaunchKernelGGL(gated_group_rmsnorm_kernel<bf16>, grid, block, 0, stream, y, ldy, z, ldz, w, eps, width / groups, (bf16*)out, ldo);
  CHECK_LAUNCH("gated_group_rmsnorm");
  return 0;
}
