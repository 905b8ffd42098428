// Linear recurrences over a matrix state per (request, head), token by token:
//     S_t = a_t S_(t-1) + b_t k_t v_t^T,   o_t = S_t^T q_t          (S: [D, E], k, q: [D], v: [E])
// in two forms that differ in where a_t and b_t come from:
//   MS_REC_DECAY: a_t = decay[head] (a constant per head), b_t = 1; o_t as above.
//   MS_REC_EXP_GATES: a log input gate i_t and a log forget gate f_t per head and token, made bounded by a soft cap,
//       i = cap tanh((x_i + bias_i) / cap), f = logsigmoid(cap tanh((x_f + bias_f) / cap)), and a running maximum
//       m_t = max(f_t + m_(t-1), i_t) (m starts at 0) that keeps the exponentials in range:
//       a_t = exp(f_t + m_(t-1) - m_t), b_t = exp(i_t - m_t); a vector n_t = a_t n_(t-1) + b_t k_t beside S;
//       o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).
//   MS_REC_WKV: a decay per key channel and token, w_t [D] (its logarithm is row t of the float32 matrix `w`, columns h D ..), and a bonus
//       u [H, D] that only the current token gets: o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t, and only then
//       S_t = diag(w_t) S_(t-1) + k_t v_t^T.
// q, k, v (and the gates' inputs) are columns of one float32 matrix x [tokens, ld] (the layer's projections);
// an activation (none or SiLU) is applied to q, k and v on the way in, q is then scaled by q_scale. Everything
// is float32. The state lives in S [slots, H, D, E] (and n [slots, H, D], m [slots, H]); a row whose
// sequence starts in this step (starts[row] == 0) begins from zero, every other row from its slot; the state after
// the row's last token is written back.
//
// One block of 256 threads per (row, head, run of EB value columns) walks the row's tokens in order with the state
// in registers (the columns of S are independent of one another, so few rows still fill the chip):
// thread (s, e) holds S[d][e] for d = s, s + NS, ... (NS = 256 / EP slices, EP the power of two that holds EB),
// adds its part of o_t[e], and the slices' parts meet in LDS in ascending s. What an output element is summed
// from, and in which order, depends on D alone: a token's result does not depend on how the sequence was
// cut into steps or batched.
#include "common.h"

#define MS_REC_DECAY 0
#define MS_REC_EXP_GATES 1
#define MS_REC_WKV 2

struct RecurrenceArgs {
  const float* x;
  int ld, q_off, k_off, v_off, i_off, f_off;
  int H, D, E, act, mode;
  float q_scale, cap;
  const float* decay;
  const void* i_bias;
  const void* f_bias;
  int bias_is_bf16;
  float* S;
  float* n;
  float* m;
  const int* row_start;
  const int* starts;
  const int* state_slots;
  float* out;
  const float* w;  // MS_REC_WKV: the decays' logarithms [tokens, ld_w], head h's D channels from column h D on
  int ld_w;
  const float* u;  // MS_REC_WKV: the bonus [H, D]
};

__device__ __forceinline__ float rec_act(float v, int act) { return act ? v / (1.f + expf(-v)) : v; }
__device__ __forceinline__ float rec_bias(const void* b, int is_bf16, int h) {
  if (b == nullptr) return 0.f;
  return is_bf16 ? to_f32(((const bf16*)b)[h]) : ((const float*)b)[h];
}
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <int PM>
__global__ __launch_bounds__(256) void gated_recurrence_kernel(RecurrenceArgs a, int EP, int EB) {
  __shared__ float qs[2][256], ks[2][256], ws[2][256], us[256];
  __shared__ float red[256];
  __shared__ float wred[2][4];
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int D = a.D, E = a.E;
  const int NS = 256 / EP, s = tid / EP;
  const int e = blockIdx.z * EB + tid % EP;  // this thread's column; columns beyond the block's run or beyond E are idle
  const bool col = tid % EP < EB && e < E;
  const int per = (D + NS - 1) / NS;
  const int t0 = a.row_start[b], t1 = a.row_start[b + 1];
  const bool fresh = a.starts[b] == 0;
  const size_t slot = (size_t)a.state_slots[b];
  float* Sg = a.S + (slot * a.H + h) * (size_t)D * E;
  const bool gates = a.mode == MS_REC_EXP_GATES, wkv = a.mode == MS_REC_WKV;
  if (wkv && tid < D) us[tid] = a.u[h * D + tid];  // read behind the first token's barrier
  float S[PM];
#pragma unroll
  for (int i = 0; i < PM; ++i) {
    const int d = s + i * NS;
    S[i] = (!fresh && i < per && d < D && col) ? Sg[(size_t)d * E + e] : 0.f;
  }
  float nv = 0.f, m = 0.f;
  if (gates && !fresh) {
    if (tid < D) nv = a.n[(slot * a.H + h) * D + tid];
    m = a.m[slot * a.H + h];
  }
  const float decay = (gates || wkv) ? 0.f : a.decay[h];
  const float bi = gates ? rec_bias(a.i_bias, a.bias_is_bf16, h) : 0.f;
  const float bf = gates ? rec_bias(a.f_bias, a.bias_is_bf16, h) : 0.f;
  for (int t = t0; t < t1; ++t) {
    const float* xr = a.x + (size_t)t * a.ld;
    const int buf = (t - t0) & 1;
    float fs = decay, is = 1.f;
    if (gates) {
      const float gi = a.cap * tanhf((xr[a.i_off + h] + bi) / a.cap);
      const float gf = log_sigmoid(a.cap * tanhf((xr[a.f_off + h] + bf) / a.cap));
      const float m_new = fmaxf(gf + m, gi);
      fs = expf(gf + m - m_new);
      is = expf(gi - m_new);
      m = m_new;
    }
    float kd = 0.f, qd = 0.f;
    if (tid < D) {
      qd = rec_act(xr[a.q_off + h * D + tid], a.act) * a.q_scale;
      kd = rec_act(xr[a.k_off + h * D + tid], a.act);
      qs[buf][tid] = qd;
      ks[buf][tid] = kd;
      if (wkv) ws[buf][tid] = expf(a.w[(size_t)t * a.ld_w + h * D + tid]);
    }
    if (gates) {
      nv = fs * nv + is * kd;  // threads beyond D carry zeros
      const float part = wave_sum(nv * qd);
      if (tid % WAVE == 0) wred[buf][tid / WAVE] = part;
    }
    const float v = col ? rec_act(xr[a.v_off + h * E + e], a.act) : 0.f;
    __syncthreads();
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < PM; ++i) {
      const int d = s + i * NS;
      if (i < per && d < D) {
        if (wkv) {
          const float kv = ks[buf][d] * v;
          acc += (S[i] + us[d] * kv) * qs[buf][d];
          S[i] = ws[buf][d] * S[i] + kv;
        } else {
          S[i] = fs * S[i] + is * ks[buf][d] * v;
          acc += S[i] * qs[buf][d];
        }
      }
    }
    if (NS > 1) {
      __syncthreads();  // the previous token's sums have been read
      red[tid] = acc;
      __syncthreads();
      if (s == 0) {
        acc = red[tid];
        for (int j = 1; j < NS; ++j) acc += red[j * EP + tid];
      }
    }
    if (s == 0 && col) {
      if (gates) {
        const float nq = (wred[buf][0] + wred[buf][1]) + (wred[buf][2] + wred[buf][3]);
        acc = acc / (fmaxf(fabsf(nq), expf(-m)) + 1e-6f);
      }
      a.out[(size_t)t * (a.H * E) + h * E + e] = acc;
    }
  }
#pragma unroll
  for (int i = 0; i < PM; ++i) {
    const int d = s + i * NS;
    if (i < per && d < D && col) Sg[(size_t)d * E + e] = S[i];
  }
  if (gates && blockIdx.z == 0) {  // every run of columns has formed the same n and m
    if (tid < D) a.n[(slot * a.H + h) * D + tid] = nv;
    if (tid == 0) a.m[slot * a.H + h] = m;
  }
}

extern "C" int ms_gated_recurrence(const float* x, int ld, int q_off, int k_off, int v_off, int i_off, int f_off, int H, int D,
                                   int E, int act, int mode, float q_scale, float cap, const float* decay, const void* i_bias,
                                   const void* f_bias, int bias_is_bf16, float* S, float* n, float* m, const int* row_start,
                                   const int* starts, const int* state_slots, float* out, int rows, const float* w, int ld_w,
                                   const float* u, hipStream_t st) {
  if (rows <= 0) return MS_OK;
  if (H <= 0 || D <= 0 || E <= 0 || x == nullptr || S == nullptr || out == nullptr || row_start == nullptr || starts == nullptr ||
      state_slots == nullptr || (act != 0 && act != 1) || q_off < 0 || k_off < 0 || v_off < 0)
    return MS_BAD_ARG;
  // (q, k and v may lie in later rows of the matrix that x is the top of: their columns are then counted past ld, and the
  // caller answers for the rows being there)
  if (mode == MS_REC_DECAY) {
    if (decay == nullptr) return MS_BAD_ARG;
  } else if (mode == MS_REC_EXP_GATES) {
    if (n == nullptr || m == nullptr || !(cap > 0.f) || i_off < 0 || f_off < 0 || i_off + H > ld || f_off + H > ld) return MS_BAD_ARG;
  } else if (mode == MS_REC_WKV) {
    if (w == nullptr || u == nullptr || ld_w < H * D) return MS_BAD_ARG;
  } else {
    return MS_BAD_ARG;
  }
  if (D > 256 || E > 256 || H > 65535) return MS_UNSUPPORTED;
  // Runs of 32 value columns, always: the order of an output's sum then depends on D alone.
  const int EB = E < 32 ? E : 32, EP = 32;
  const int per = (D + 256 / EP - 1) / (256 / EP);
  RecurrenceArgs a{x, ld, q_off, k_off, v_off, i_off, f_off, H, D, E, act, mode, q_scale, cap, decay, i_bias, f_bias, bias_is_bf16,
                   S, n, m, row_start, starts, state_slots, out, w, ld_w, u};
  const dim3 grid(rows, H, (E + EB - 1) / EB);
  if (per <= 4) gated_recurrence_kernel<4><<<grid, 256, 0, st>>>(a, EP, EB);
  else if (per <= 16) gated_recurrence_kernel<16><<<grid, 256, 0, st>>>(a, EP, EB);
  else if (per <= 64) gated_recurrence_kernel<64><<<grid, 256, 0, st>>>(a, EP, EB);
  else if (per <= 128) gated_recurrence_kernel<128><<<grid, 256, 0, st>>>(a, EP, EB);
  else return MS_UNSUPPORTED;
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// The same recurrences for rows that bring many tokens, in chunks of REC_CHUNK tokens and three passes, so
// that the work is matrix products over a chunk and every chunk of every row and head has a block of its own:
//   1. per chunk: the chunk's own contribution to the state at its end, U = sum_j w_j k_j v_j^T (and u = sum_j
//      w_j k_j), w_j = exp(B - b_j + i_j - a) with b_j the log forget gates summed from the chunk's start through
//      j, B = b_last, and a = max_j (B - b_j + i_j) (a = 0 for the constant decay, whose weights cannot grow);
//   2. per (row, head), chunk after chunk: m' = max(B + m, a), S' = exp(B + m - m') S + exp(a - m') U; the state
//      *before* each chunk takes U's place in the buffer, m and n before it are kept beside it; the state after
//      the last chunk goes to the slot;
//   3. per chunk: with the state S0 (n0, m0) before it, m_t by its own recurrence from m0,
//      o_t = g_t S0^T q_t + sum_(j <= t) P_tj v_j,  P_tj = (q_t . k_j) exp(b_t - b_j + i_j - m_t),  g_t = exp(b_t + m0 - m_t),
//      n_t . q_t = g_t n0 . q_t + sum_j P_tj, and the normaliser as above.
// Every exponent is at most zero by the definition of the maxima. All float32; sums are reassociated against the
// token-by-token kernel, nothing else differs. Head sizes up to REC_CHUNK_MAX_DIM; larger ones take the other kernel.
#define REC_CHUNK 64
#define REC_CHUNK_MAX_DIM 128

struct ChunkArgs {
  RecurrenceArgs r;
  float* U;    // [chunks, H, D * E]
  float* u;    // [chunks, H, D]
  double* cs;  // [chunks, H, 4]: B, a, m before the chunk (double: B may be in the hundreds where B + m is small)
  int rows;
};

// The chunk `c` of the step: its row, first token and token count; *base = index of the row's first chunk.
__device__ __forceinline__ void find_chunk(const int* __restrict__ row_start, int rows, int c, int* row, int* first, int* count,
                                           int* base) {
  int b = 0, at = 0;
  for (; b < rows - 1; ++b) {
    const int nc = (row_start[b + 1] - row_start[b] + REC_CHUNK - 1) / REC_CHUNK;
    if (c < at + nc) break;
    at += nc;
  }
  *row = b;
  *base = at;
  *first = row_start[b] + (c - at) * REC_CHUNK;
  const int left = row_start[b + 1] - *first;
  *count = left < REC_CHUNK ? left : REC_CHUNK;
}

// Log gates of the chunk's tokens into gi[] (and fg[], if given), and the running sums of the log forget gates into
// bs[] (thread 0 adds). The sums are kept in double precision: the kernels need their differences, which may be small
// where the sums are in the hundreds, and in float32 such a difference would carry the sums' rounding.
__device__ __forceinline__ void chunk_gates(const RecurrenceArgs& a, int h, int first, int count, float* gi, double* bs,
                                            float* fg = nullptr) {
  const int tid = threadIdx.x;
  if (tid < REC_CHUNK) {
    float i = 0.f, f = 0.f;
    if (tid < count) {
      if (a.mode == MS_REC_EXP_GATES) {
        const float* xr = a.x + (size_t)(first + tid) * a.ld;
        i = a.cap * tanhf((xr[a.i_off + h] + rec_bias(a.i_bias, a.bias_is_bf16, h)) / a.cap);
        f = log_sigmoid(a.cap * tanhf((xr[a.f_off + h] + rec_bias(a.f_bias, a.bias_is_bf16, h)) / a.cap));
      } else {
        f = logf(a.decay[h]);
      }
    }
    gi[tid] = i;
    bs[tid] = (double)f;
    if (fg != nullptr) fg[tid] = f;
  }
  __syncthreads();
  if (tid == 0) {
    double run = 0.0;
    for (int j = 0; j < REC_CHUNK; ++j) {
      run += bs[j];
      bs[j] = run;
    }
  }
  __syncthreads();
}

__global__ __launch_bounds__(256) void rec_chunk_summary_kernel(ChunkArgs c) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const RecurrenceArgs& a = c.r;
  const int D = a.D, E = a.E, h = blockIdx.y, tid = threadIdx.x;
  const int DP = (D + 3) & ~3, EP = (E + 3) & ~3;
  float* Kw = sm;                    // [REC_CHUNK][DP], keys times their weights
  float* V = Kw + REC_CHUNK * DP;    // [REC_CHUNK][EP]
  float* gi = V + REC_CHUNK * EP;    // [REC_CHUNK]
  float* wt = gi + REC_CHUNK;        // [REC_CHUNK]
  __shared__ double bs[REC_CHUNK];
  __shared__ float amax;
  int row, first, count, base;
  find_chunk(a.row_start, c.rows, blockIdx.x, &row, &first, &count, &base);
  chunk_gates(a, h, first, count, gi, bs);
  const double B = bs[count - 1];
  const bool gates = a.mode == MS_REC_EXP_GATES;
  if (tid == 0) {
    float mx = 0.f;
    if (gates) {
      mx = -INFINITY;
      for (int j = 0; j < count; ++j) mx = fmaxf(mx, (float)(B - bs[j]) + gi[j]);
    }
    amax = mx;
  }
  __syncthreads();
  if (tid < REC_CHUNK) wt[tid] = tid < count ? expf((float)(B - bs[tid]) + gi[tid] - amax) : 0.f;
  __syncthreads();
  for (int i = tid; i < REC_CHUNK * DP; i += 256) {
    const int j = i / DP, d = i % DP;
    Kw[i] = (j < count && d < D) ? wt[j] * rec_act(a.x[(size_t)(first + j) * a.ld + a.k_off + h * D + d], a.act) : 0.f;
  }
  for (int i = tid; i < REC_CHUNK * EP; i += 256) {
    const int j = i / EP, e = i % EP;
    V[i] = (j < count && e < E) ? rec_act(a.x[(size_t)(first + j) * a.ld + a.v_off + h * E + e], a.act) : 0.f;
  }
  __syncthreads();
  // thread: 8 rows d0.. of U by 8 columns e0..
  const int d0 = (tid / 16) * 8, e0 = (tid % 16) * 8;
  float acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[i][k] = 0.f;
  if (d0 < DP && e0 < EP) {
#pragma unroll 2
    for (int j = 0; j < count; ++j) {
      float kd[8], ve[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) kd[i] = d0 + i < DP ? Kw[j * DP + d0 + i] : 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) ve[k] = e0 + k < EP ? V[j * EP + e0 + k] : 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[i][k] = fmaf(kd[i], ve[k], acc[i][k]);
    }
  }
  float* Uo = c.U + ((size_t)blockIdx.x * a.H + h) * D * E;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (d0 + i < D && e0 + k < E) Uo[(size_t)(d0 + i) * E + e0 + k] = acc[i][k];
  if (gates && tid < D) {
    float s = 0.f;
    for (int j = 0; j < count; ++j) s += Kw[j * DP + tid];
    c.u[((size_t)blockIdx.x * a.H + h) * D + tid] = s;
  }
  if (tid == 0) {
    double* o = c.cs + ((size_t)blockIdx.x * a.H + h) * 4;
    o[0] = B;
    o[1] = (double)amax;
  }
}

// Pass 2. grid (rows, H, slices): a block owns every slices-th run of 256 elements of the state.
__global__ __launch_bounds__(256) void rec_chunk_scan_kernel(ChunkArgs c, int slices) {
  const RecurrenceArgs& a = c.r;
  const int b = blockIdx.x, h = blockIdx.y, z = blockIdx.z, tid = threadIdx.x;
  const int DE = a.D * a.E;
  int base = 0;
  for (int r = 0; r < b; ++r) base += (a.row_start[r + 1] - a.row_start[r] + REC_CHUNK - 1) / REC_CHUNK;
  const int nc = (a.row_start[b + 1] - a.row_start[b] + REC_CHUNK - 1) / REC_CHUNK;
  const bool fresh = a.starts[b] == 0;
  const bool gates = a.mode == MS_REC_EXP_GATES;
  const size_t slot = (size_t)a.state_slots[b];
  float* Sg = a.S + (slot * a.H + h) * (size_t)DE;
  constexpr int PER = 8;
  float S[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = (z + slices * i) * 256 + tid;
    S[i] = (!fresh && idx < DE) ? Sg[idx] : 0.f;
  }
  const bool own_n = gates && z == 0 && tid < a.D;
  float nv = (own_n && !fresh) ? a.n[(slot * a.H + h) * a.D + tid] : 0.f;
  double m = (gates && !fresh) ? (double)a.m[slot * a.H + h] : 0.0;
  for (int k = 0; k < nc; ++k) {
    const size_t at = (size_t)(base + k) * a.H + h;
    float* Uc = c.U + at * DE;
    double* csk = c.cs + at * 4;
    const double B = csk[0], amax = csk[1];
    float alpha, beta;
    if (gates) {
      const double m_new = fmax(B + m, amax);
      alpha = expf((float)(B + m - m_new));
      beta = expf((float)(amax - m_new));
      if (z == 0 && tid == 0) csk[2] = m;
      m = m_new;
    } else {
      alpha = expf((float)B);
      beta = 1.f;
    }
    float t[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = (z + slices * i) * 256 + tid;
      t[i] = idx < DE ? Uc[idx] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = (z + slices * i) * 256 + tid;
      if (idx < DE) Uc[idx] = S[i];
      S[i] = alpha * S[i] + beta * t[i];
    }
    if (own_n) {
      float* uc = c.u + at * a.D;
      const float t2 = uc[tid];
      uc[tid] = nv;
      nv = alpha * nv + beta * t2;
    }
  }
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = (z + slices * i) * 256 + tid;
    if (idx < DE) Sg[idx] = S[i];
  }
  if (own_n) a.n[(slot * a.H + h) * a.D + tid] = nv;
  if (gates && z == 0 && tid == 0) a.m[slot * a.H + h] = (float)m;
}

__global__ __launch_bounds__(256) void rec_chunk_output_kernel(ChunkArgs c) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const RecurrenceArgs& a = c.r;
  const int D = a.D, E = a.E, h = blockIdx.y, tid = threadIdx.x;
  const int DQ = D | 1;              // odd row stride: rows of Q fall into different banks
  const int EP = (E + 3) & ~3;
  constexpr int CP = REC_CHUNK + 1;
  float* V = sm;                     // [REC_CHUNK][EP], first: it is read four floats at a time
  float* Q = V + REC_CHUNK * EP;     // [REC_CHUNK][DQ]
  float* Kt = Q + REC_CHUNK * DQ;    // [D][CP], keys transposed
  float* P = Kt + D * CP;            // [REC_CHUNK][CP]
  float* gi = P + REC_CHUNK * CP;    // [REC_CHUNK]
  float* mt = gi + REC_CHUNK;
  float* nq = mt + REC_CHUNK;
  float* fg = nq + REC_CHUNK;
  float* n0 = fg + REC_CHUNK;        // [D]
  __shared__ double bs[REC_CHUNK];
  int row, first, count, base;
  find_chunk(a.row_start, c.rows, blockIdx.x, &row, &first, &count, &base);
  chunk_gates(a, h, first, count, gi, bs, fg);
  const bool gates = a.mode == MS_REC_EXP_GATES;
  const size_t at = (size_t)blockIdx.x * a.H + h;
  const double m0 = gates ? c.cs[at * 4 + 2] : 0.0;
  if (tid == 0) {
    float m = (float)m0;  // the running maximum by its own recurrence, as the token-by-token kernel forms it
    for (int j = 0; j < REC_CHUNK; ++j) {
      if (gates && j < count) m = fmaxf(fg[j] + m, gi[j]);
      mt[j] = m;
    }
  }
  for (int i = tid; i < REC_CHUNK * D; i += 256) {
    const int j = i / D, d = i % D;
    const bool in = j < count;
    const float* xr = a.x + (size_t)(first + (in ? j : 0)) * a.ld;
    Q[j * DQ + d] = in ? rec_act(xr[a.q_off + h * D + d], a.act) * a.q_scale : 0.f;
    Kt[d * CP + j] = in ? rec_act(xr[a.k_off + h * D + d], a.act) : 0.f;
  }
  for (int i = tid; i < REC_CHUNK * EP; i += 256) {
    const int j = i / EP, e = i % EP;
    V[i] = (j < count && e < E) ? rec_act(a.x[(size_t)(first + j) * a.ld + a.v_off + h * E + e], a.act) : 0.f;
  }
  if (gates && tid < D) n0[tid] = c.u[at * D + tid];
  __syncthreads();
  {
    // scores: thread = 4 tokens t0.. by 4 keys j0..
    const int t0 = (tid / 16) * 4, j0 = (tid % 16) * 4;
    float s[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int k = 0; k < 4; ++k) s[i][k] = 0.f;
    if (j0 <= t0 + 3) {  // blocks wholly above the diagonal stay zero
#pragma unroll 4
      for (int d = 0; d < D; ++d) {
        float qv[4], kv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) qv[i] = Q[(t0 + i) * DQ + d];
#pragma unroll
        for (int k = 0; k < 4; ++k) kv[k] = Kt[d * CP + j0 + k];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int k = 0; k < 4; ++k) s[i][k] = fmaf(qv[i], kv[k], s[i][k]);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int t = t0 + i, j = j0 + k;
        P[t * CP + j] = (j <= t && t < count) ? s[i][k] * expf((float)(bs[t] - bs[j]) + gi[j] - mt[t]) : 0.f;
      }
  }
  __syncthreads();
  if (gates && tid < REC_CHUNK) {
    float sum = 0.f;
    for (int j = 0; j <= tid; ++j) sum += P[tid * CP + j];
    float dot = 0.f;
    for (int d = 0; d < D; ++d) dot = fmaf(n0[d], Q[tid * DQ + d], dot);
    nq[tid] = expf((float)(bs[tid] + m0 - (double)mt[tid])) * dot + sum;
  }
  // outputs: thread = 8 tokens t0.. by 4 columns e0..
  const int t0 = (tid / 32) * 8, e0 = (tid % 32) * 4;
  float o[8][4], in[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int k = 0; k < 4; ++k) o[i][k] = in[i][k] = 0.f;
  if (e0 < EP) {
    const float* S0 = c.U + at * (size_t)D * E;
    const bool vec = (E % 4) == 0;
#pragma unroll 4
    for (int d = 0; d < D; ++d) {
      float sv[4];
      if (vec) {
        const float4 v4 = *reinterpret_cast<const float4*>(S0 + (size_t)d * E + e0);
        sv[0] = v4.x; sv[1] = v4.y; sv[2] = v4.z; sv[3] = v4.w;
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) sv[k] = e0 + k < E ? S0[(size_t)d * E + e0 + k] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float qv = Q[(t0 + i) * DQ + d];
#pragma unroll
        for (int k = 0; k < 4; ++k) in[i][k] = fmaf(qv, sv[k], in[i][k]);
      }
    }
    const int jend = t0 + 8 < count ? t0 + 8 : count;
#pragma unroll 4
    for (int j = 0; j < jend; ++j) {
      const float4 v4 = *reinterpret_cast<const float4*>(V + j * EP + e0);
      const float vv[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float p = P[(t0 + i) * CP + j];
#pragma unroll
        for (int k = 0; k < 4; ++k) o[i][k] = fmaf(p, vv[k], o[i][k]);
      }
    }
  }
  __syncthreads();  // nq is complete
  if (e0 < EP) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int t = t0 + i;
      if (t >= count) continue;
      const float g = expf((float)(bs[t] + m0 - (double)mt[t]));
      const float den = gates ? fmaxf(fabsf(nq[t]), expf(-mt[t])) + 1e-6f : 1.f;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (e0 + k < E) a.out[(size_t)(first + t) * (a.H * E) + h * E + e0 + k] = (g * in[i][k] + o[i][k]) / den;
    }
  }
}

static size_t summary_lds(int D, int E) { return sizeof(float) * ((size_t)REC_CHUNK * (((D + 3) & ~3) + ((E + 3) & ~3)) + 2 * REC_CHUNK); }
static size_t output_lds(int D, int E) {
  return sizeof(float) * ((size_t)REC_CHUNK * (D | 1) + (size_t)D * (REC_CHUNK + 1) + (size_t)REC_CHUNK * ((E + 3) & ~3) +
                          (size_t)REC_CHUNK * (REC_CHUNK + 1) + 4 * REC_CHUNK + D);
}

// Floats of scratch per chunk and head that ms_gated_recurrence_chunked needs for U; u takes D and cs 4 per chunk and head.
extern "C" int ms_gated_recurrence_chunk_tokens() { return REC_CHUNK; }
extern "C" int ms_gated_recurrence_chunk_max_dim() { return REC_CHUNK_MAX_DIM; }

// As ms_gated_recurrence, in chunks. `chunks` = sum over the rows of ceil(tokens / REC_CHUNK) (the host knows the rows'
// lengths); U [chunks, H, D * E], u [chunks, H, D] (float) and cs [chunks, H, 4] (double) are scratch.
extern "C" int ms_gated_recurrence_chunked(const float* x, int ld, int q_off, int k_off, int v_off, int i_off, int f_off, int H, int D,
                                           int E, int act, int mode, float q_scale, float cap, const float* decay,
                                           const void* i_bias, const void* f_bias, int bias_is_bf16, float* S, float* n, float* m,
                                           const int* row_start, const int* starts, const int* state_slots, float* out, int rows,
                                           int chunks, float* U, float* u, double* cs, hipStream_t st) {
  if (rows <= 0 || chunks <= 0) return MS_OK;
  if (H <= 0 || D <= 0 || E <= 0 || x == nullptr || S == nullptr || out == nullptr || row_start == nullptr || starts == nullptr ||
      state_slots == nullptr || U == nullptr || cs == nullptr || (act != 0 && act != 1) || q_off < 0 || k_off < 0 || v_off < 0 ||
      q_off + H * D > ld || k_off + H * D > ld || v_off + H * E > ld)
    return MS_BAD_ARG;
  if (mode == MS_REC_DECAY) {
    if (decay == nullptr) return MS_BAD_ARG;
  } else if (mode == MS_REC_EXP_GATES) {
    if (n == nullptr || m == nullptr || u == nullptr || !(cap > 0.f) || i_off < 0 || f_off < 0 || i_off + H > ld || f_off + H > ld)
      return MS_BAD_ARG;
  } else {
    return MS_BAD_ARG;
  }
  if (D > REC_CHUNK_MAX_DIM || E > REC_CHUNK_MAX_DIM || H > 65535 || rows > 65535) return MS_UNSUPPORTED;
  ChunkArgs c{{x, ld, q_off, k_off, v_off, i_off, f_off, H, D, E, act, mode, q_scale, cap, decay, i_bias, f_bias, bias_is_bf16, S, n,
               m, row_start, starts, state_slots, out},
              U, u, cs, rows};
  const size_t lds1 = summary_lds(D, E), lds3 = output_lds(D, E);
  if (hipFuncSetAttribute((const void*)rec_chunk_summary_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds1) != hipSuccess ||
      hipFuncSetAttribute((const void*)rec_chunk_output_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds3) != hipSuccess)
    return MS_LAUNCH_FAILED;
  rec_chunk_summary_kernel<<<dim3(chunks, H), 256, lds1, st>>>(c);
  const int slices = (D * E + 256 * 8 - 1) / (256 * 8);
  rec_chunk_scan_kernel<<<dim3(rows, H, slices), 256, 0, st>>>(c, slices);
  rec_chunk_output_kernel<<<dim3(chunks, H), 256, lds3, st>>>(c);
  return launch_status();
}
