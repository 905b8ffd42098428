// Norms beyond the plain RMSNorm, all with float32 statistics and one rounding at the store:
//   layer norm with weight and bias (optionally over a list of rows);
//   RMS norm over groups of a row, times a weight, times sigmoid(gate) (a gated output norm: one group per head,
//   or one group for the whole row);
//   the mean of several streams, each RMS-normed over the row with its own weight, added to the residual stream;
//   a scale in place;
//   RMS norm of the whole query projection and of the whole key projection of a token (before they are split into
//   heads), rotation of part of every head, and the store of keys and values into the cache pages.
#include "common.h"

// ---------------------------------------------------------------------------------------------
// y[r, :] = (x[row(r), :] - mean) * rsqrt(var + eps) * w + b, var = mean of squared deviations.
// One block per row. Mean first, then the deviations' squares: two passes over the row, of which a thread keeps
// its first eight elements in registers. Sums per thread in ascending element order, then a fixed block order.
template <typename TW, typename TO, int NT>
__global__ __launch_bounds__(NT) void layernorm_kernel(const float* __restrict__ x, const TW* __restrict__ w,
                                                       const TW* __restrict__ b, TO* __restrict__ y,
                                                       const int* __restrict__ rows, int width, float eps) {
  __shared__ float red[NT / WAVE];
  constexpr int KEEP = 8;  // elements a thread keeps in registers between the passes (wider rows are read again)
  const int r = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * width;
  float kept[KEEP];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int e = threadIdx.x + i * NT;
    kept[i] = e < width ? xr[e] : 0.f;
    s += kept[i];
  }
  for (int e = threadIdx.x + KEEP * NT; e < width; e += NT) s += xr[e];
  const float mean = block_sum<NT>(s, red) / (float)width;
  float v = 0.f;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const float d = kept[i] - mean;
    if (threadIdx.x + i * NT < width) v += d * d;
  }
  for (int e = threadIdx.x + KEEP * NT; e < width; e += NT) {
    const float d = xr[e] - mean;
    v += d * d;
  }
  const float rstd = 1.f / sqrtf(block_sum<NT>(v, red) / (float)width + eps);
  TO* yr = y + (size_t)r * width;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int e = threadIdx.x + i * NT;
    if (e < width) {
      float o = (kept[i] - mean) * rstd * to_f32(w[e]);
      if (b != nullptr) o += to_f32(b[e]);
      yr[e] = from_f32<TO>(o);
    }
  }
  for (int e = threadIdx.x + KEEP * NT; e < width; e += NT) {
    float o = (xr[e] - mean) * rstd * to_f32(w[e]);
    if (b != nullptr) o += to_f32(b[e]);
    yr[e] = from_f32<TO>(o);
  }
}

extern "C" int ms_layernorm(const float* x, const void* w, const void* b, int w_is_bf16, void* y, int y_is_bf16,
                            const int* rows, int n_rows, int width, float eps, hipStream_t st) {
  if (n_rows <= 0) return MS_OK;
  if (width <= 0 || !(eps >= 0.f)) return MS_BAD_ARG;
#define LN(TW, TO) layernorm_kernel<TW, TO, 256><<<n_rows, 256, 0, st>>>(x, (const TW*)w, (const TW*)b, (TO*)y, rows, width, eps)
  if (w_is_bf16) { if (y_is_bf16) LN(bf16, bf16); else LN(bf16, float); }
  else { if (y_is_bf16) LN(float, bf16); else LN(float, float); }
#undef LN
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// y[t, g * group + e] = x[t, g * group + e] * rsqrt(mean over the group of x^2 + eps) * w[g * group + e]
//                       * sigmoid(gate[t * gate_stride + g * group + e])     (gate_act = 1: SiLU instead of the sigmoid)
// w == nullptr: no weight; gate == nullptr: no gate. One wave per (token, group) when the group is at
// most 256 wide (four groups per block), else one block per (token, group).
template <typename TW, typename TO>
__global__ __launch_bounds__(256) void group_rmsnorm_gate_kernel(const float* __restrict__ x, const TW* __restrict__ w,
                                                                 const float* __restrict__ gate, int gate_stride,
                                                                 TO* __restrict__ y, int groups, int group, float eps,
                                                                 int per_wave, int gate_act) {
  __shared__ float red[256 / WAVE];
  const int t = blockIdx.x;
  const int width = groups * group;
  int g, first, step;
  if (per_wave) {
    g = blockIdx.y * 4 + threadIdx.x / WAVE;
    first = threadIdx.x % WAVE;
    step = WAVE;
  } else {
    g = blockIdx.y;
    first = threadIdx.x;
    step = 256;
  }
  const bool live = g < groups;
  const float* xr = x + (size_t)t * width + (size_t)(live ? g : 0) * group;
  float s = 0.f;
  if (live)
    for (int e = first; e < group; e += step) s += xr[e] * xr[e];
  s = per_wave ? wave_sum(s) : block_sum<256>(s, red);
  if (!live) return;
  const float rstd = 1.f / sqrtf(s / (float)group + eps);
  for (int e = first; e < group; e += step) {
    const int c = g * group + e;
    float o = xr[e] * rstd;
    if (w != nullptr) o *= to_f32(w[c]);
    if (gate != nullptr) {
      const float z = gate[(size_t)t * gate_stride + c];
      o *= (gate_act ? z : 1.f) / (1.f + expf(-z));  // sigmoid(z), or z sigmoid(z)
    }
    y[(size_t)t * width + c] = from_f32<TO>(o);
  }
}

extern "C" int ms_group_rmsnorm_gate(const float* x, const void* w, int w_is_bf16, const float* gate, int gate_stride,
                                     void* y, int y_is_bf16, int tokens, int groups, int group, float eps, int gate_act,
                                     hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if ((gate_act != 0 && gate_act != 1) || groups <= 0 || group <= 0 || tokens > 65535 * 32 || !(eps >= 0.f) || (gate != nullptr && gate_stride < groups * group))
    return MS_BAD_ARG;
  const int per_wave = group <= 256;
  const dim3 grid(tokens, per_wave ? (groups + 3) / 4 : groups);
  if (grid.y > 65535) return MS_UNSUPPORTED;
#define GN(TW, TO) group_rmsnorm_gate_kernel<TW, TO><<<grid, 256, 0, st>>>(x, (const TW*)w, gate, gate_stride, (TO*)y, groups, group, eps, per_wave, gate_act)
  if (w_is_bf16) { if (y_is_bf16) GN(bf16, bf16); else GN(bf16, float); }
  else { if (y_is_bf16) GN(float, bf16); else GN(float, float); }
#undef GN
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// residual[t, :] += coef * sum over the n streams i of ( s_i[t, :] * rsqrt(mean(s_i[t]^2) + eps) * w_i ), the
// streams' terms added in ascending i before the sum meets the residual. n <= 4. One block per token.
struct NormedStreams {
  const float* s[4];
  const void* w[4];
};

template <typename TW>
__global__ __launch_bounds__(256) void normed_mean_add_kernel(float* __restrict__ residual, NormedStreams in, int n, int width,
                                                              float eps, float coef) {
  __shared__ float red[256 / WAVE];
  const int t = blockIdx.x;
  float rstd[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (i >= n) break;  // n is the same for all threads
    const float* sr = in.s[i] + (size_t)t * width;
    float ss = 0.f;
    for (int e = threadIdx.x; e < width; e += 256) ss += sr[e] * sr[e];
    rstd[i] = 1.f / sqrtf(block_sum<256>(ss, red) / (float)width + eps);
  }
  for (int e = threadIdx.x; e < width; e += 256) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < n) acc += in.s[i][(size_t)t * width + e] * rstd[i] * to_f32(((const TW*)in.w[i])[e]);
    residual[(size_t)t * width + e] += coef * acc;
  }
}

extern "C" int ms_normed_mean_add(float* residual, const float* const* streams, const void* const* weights, int w_is_bf16, int n,
                                  int tokens, int width, float eps, float coef, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (n < 1 || n > 4 || width <= 0 || !(eps >= 0.f)) return MS_BAD_ARG;
  NormedStreams in;
  for (int i = 0; i < 4; ++i) {
    in.s[i] = i < n ? streams[i] : nullptr;
    in.w[i] = i < n ? weights[i] : nullptr;
  }
  if (w_is_bf16) normed_mean_add_kernel<bf16><<<tokens, 256, 0, st>>>(residual, in, n, width, eps, coef);
  else normed_mean_add_kernel<float><<<tokens, 256, 0, st>>>(residual, in, n, width, eps, coef);
  return launch_status();
}

// residual += rmsnorm(stream + pending) * w for one stream whose last matrix product may have left partial sums (`splits`
// slices `stride` floats apart, added in ascending order; parts may be nullptr): the sums are formed inside the norm
// instead of being written out by a kernel of their own. A block of 1,024 threads per row; a thread keeps the sums of its
// first eight elements in registers between the mean of squares and the result (rows up to 8,192 wide are summed once;
// what lies beyond is summed again). stream may be nullptr (zero). What the next reader of the residual would otherwise
// launch kernels for can ride along: `next` (bfloat16, nullable) receives the new residual rounded, and with `clear` the
// stream is left zero for the next sublayer to add into.
template <typename TW>
__global__ __launch_bounds__(1024) void normed_add_pending_kernel(float* __restrict__ residual, float* __restrict__ stream,
                                                                  const float* __restrict__ parts, int splits, size_t stride,
                                                                  const TW* __restrict__ w, int width, float eps,
                                                                  bf16* __restrict__ next, int clear) {
  constexpr int NT = 1024, KEPT = 8;
  __shared__ float red[NT / WAVE];
  const size_t row = (size_t)blockIdx.x * width;
  float kept[KEPT];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < KEPT; ++i) {
    const int e = threadIdx.x + i * NT;
    kept[i] = e < width ? (stream ? stream[row + e] : 0.f) + (parts ? sum_splits(parts + row + e, splits, stride) : 0.f) : 0.f;
    ss += kept[i] * kept[i];
  }
  for (int e = threadIdx.x + KEPT * NT; e < width; e += NT) {
    const float v = (stream ? stream[row + e] : 0.f) + (parts ? sum_splits(parts + row + e, splits, stride) : 0.f);
    ss += v * v;
  }
  const float rstd = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < KEPT; ++i) {
    const int e = threadIdx.x + i * NT;
    if (e < width) {
      const float r = residual[row + e] + kept[i] * rstd * to_f32(w[e]);
      residual[row + e] = r;
      if (next) next[row + e] = static_cast<bf16>(r);
      if (clear && stream) stream[row + e] = 0.f;
    }
  }
  for (int e = threadIdx.x + KEPT * NT; e < width; e += NT) {
    const float v = (stream ? stream[row + e] : 0.f) + (parts ? sum_splits(parts + row + e, splits, stride) : 0.f);
    const float r = residual[row + e] + v * rstd * to_f32(w[e]);
    residual[row + e] = r;
    if (next) next[row + e] = static_cast<bf16>(r);
    if (clear && stream) stream[row + e] = 0.f;
  }
}

extern "C" int ms_normed_add_pending(float* residual, float* stream, const float* parts, int splits, long long stride,
                                     const void* w, int w_is_bf16, int tokens, int width, float eps, void* next_bf16, int clear,
                                     hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (width <= 0 || (parts == nullptr && stream == nullptr) || !(eps >= 0.f)) return MS_BAD_ARG;
  if (parts != nullptr && (splits < 1 || stride < (long long)tokens * width)) return MS_BAD_ARG;
  if (w_is_bf16) normed_add_pending_kernel<bf16><<<tokens, 1024, 0, st>>>(residual, stream, parts, splits, (size_t)stride, (const bf16*)w, width, eps, (bf16*)next_bf16, clear);
  else normed_add_pending_kernel<float><<<tokens, 1024, 0, st>>>(residual, stream, parts, splits, (size_t)stride, (const float*)w, width, eps, (bf16*)next_bf16, clear);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
__global__ void scale_kernel(float* __restrict__ x, size_t n, float s) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] *= s;
}

extern "C" int ms_scale(float* x, long long n, float s, hipStream_t st) {
  if (n <= 0) return MS_OK;
  scale_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(x, (size_t)n, s);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// A token's row of qkv (float32, row stride ld) holds Hq * D query elements, then Hkv * D key elements, then
// Hkv * Dv value elements.
//   q, k: optional RMS norm over the whole query part / the whole key part (weights [Hq * D], [Hkv * D]; nullptr:
//         none), then rotation of the first `rot` elements of every head in pairs, (j, j + rot/2) or (2j, 2j + 1), by
//         the angle whose cosine and sine are rope[t][j] and rope[t][rot/2 + j];
//   q goes to q_out [tokens, Hq * D]; k and v go to the cache page of the token's slot (keys
//   [pages, Hkv, page_size, D], values transposed within the page, [pages, Hkv, Dv, page_size]).
// slots == nullptr: only the queries. One block per token. bias (optional, the row's columns) is added to the projection
// before anything else; the values are the Hkv * Dv columns from v_col on (behind the keys, or the key columns themselves:
// values that are the keys as projected, before norm and rotation).
template <typename T, typename TW>
__global__ __launch_bounds__(256) void qkv_norm_rope_store_kernel(
    const float* __restrict__ qkv, int ld, T* __restrict__ q_out, const int* __restrict__ slots, const TW* __restrict__ qw,
    const TW* __restrict__ kw, const TW* __restrict__ bias, int v_col, float eps, const float* __restrict__ rope, int rot,
    int pairing, T* __restrict__ kc, T* __restrict__ vc, int Hq, int Hkv, int D, int Dv, int page_size) {
  __shared__ float red[256 / WAVE];
  const int t = blockIdx.x;
  const float* row = qkv + (size_t)t * ld;
  const int nq = Hq * D, nk = Hkv * D, nv = Hkv * Dv;
  const int half = rot / 2;
  const float* cs = rot > 0 ? rope + (size_t)t * rot : nullptr;
  const int s = slots ? slots[t] : 0;
  for (int part = 0; part < (slots ? 2 : 1); ++part) {
    const int c0 = part ? nq : 0;  // the part's first column: the bias has the row's columns
    const float* src = row + c0;
    const TW* b = bias ? bias + c0 : nullptr;
    const int n = part ? nk : nq;
    const TW* w = part ? kw : qw;
    float rstd = 1.f;
    if (w != nullptr) {
      float ss = 0.f;
      for (int e = threadIdx.x; e < n; e += 256) {
        const float x = src[e] + (b ? to_f32(b[e]) : 0.f);
        ss += x * x;
      }
      rstd = 1.f / sqrtf(block_sum<256>(ss, red) / (float)n + eps);
    }
    for (int e = threadIdx.x; e < n; e += 256) {
      const int h = e / D, d = e % D;
      float v = (src[e] + (b ? to_f32(b[e]) : 0.f)) * rstd * (w ? to_f32(w[e]) : 1.f);
      if (d < rot) {
        const bool first = pairing == MS_ROPE_ADJACENT ? (d & 1) == 0 : d < half;
        const int j = pairing == MS_ROPE_ADJACENT ? d / 2 : (d < half ? d : d - half);
        const int pe = e - d + (pairing == MS_ROPE_ADJACENT ? (d ^ 1) : (d < half ? d + half : d - half));
        const float p = (src[pe] + (b ? to_f32(b[pe]) : 0.f)) * rstd * (w ? to_f32(w[pe]) : 1.f);
        v = first ? v * cs[j] - p * cs[half + j] : v * cs[j] + p * cs[half + j];
      }
      if (part == 0) q_out[(size_t)t * nq + e] = from_f32<T>(v);
      else kc[(((size_t)(s / page_size) * Hkv + h) * page_size + (s % page_size)) * D + d] = from_f32<T>(v);
    }
  }
  if (slots) {
    const float* src = row + v_col;
    for (int e = threadIdx.x; e < nv; e += 256) {
      const int h = e / Dv, d = e % Dv;
      const float v = src[e] + (bias ? to_f32(bias[v_col + e]) : 0.f);
      vc[(((size_t)(s / page_size) * Hkv + h) * Dv + d) * page_size + (s % page_size)] = from_f32<T>(v);
    }
  }
}

extern "C" int ms_qkv_norm_rope_store(const float* qkv, int ld, void* q_out, int is_bf16, const int* slots, const void* qw,
                                      const void* kw, const void* bias, int v_col, int w_is_bf16, float eps, const float* rope,
                                      int rot, int pairing, void* kc, void* vc, int tokens, int Hq, int Hkv, int D, int Dv,
                                      int page_size, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (Hq <= 0 || Hkv <= 0 || D <= 0 || Dv <= 0 || page_size <= 0 || rot < 0 || rot > D || rot % 2 || (rot > 0 && rope == nullptr) ||
      ld < Hq * D + (slots ? Hkv * D : 0) || (slots != nullptr && (kc == nullptr || vc == nullptr || v_col < 0 || v_col + Hkv * Dv > ld)) ||
      (qw == nullptr) != (kw == nullptr) || !(eps >= 0.f))
    return MS_BAD_ARG;
  if (pairing != MS_ROPE_HALVES && pairing != MS_ROPE_ADJACENT) return MS_UNSUPPORTED;
#define QK(T, TW) qkv_norm_rope_store_kernel<T, TW><<<tokens, 256, 0, st>>>(qkv, ld, (T*)q_out, slots, (const TW*)qw, (const TW*)kw, (const TW*)bias, v_col, eps, rope, rot, pairing, (T*)kc, (T*)vc, Hq, Hkv, D, Dv, page_size)
  if (is_bf16) { if (w_is_bf16) QK(bf16, bf16); else QK(bf16, float); }
  else { if (w_is_bf16) QK(float, bf16); else QK(float, float); }
#undef QK
  return launch_status();
}
