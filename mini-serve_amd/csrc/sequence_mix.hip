// What stands between a mixer's fused projection and its attention kernel, for mixers whose queries, keys and values
// are not plain slices of the projection: a short causal convolution over time with per-head norms, and the
// preparation of a latent attention (one small vector per token from which every head's keys and values derive).
// Everything here is float32 arithmetic on a float32 projection; what is stored (queries, cache) is rounded once.
#include "common.h"

// ---------------------------------------------------------------------------------------------
// Short causal convolution over time on every channel of a token's projection row, then an RMS norm per group of D
// channels of the query part and of the key part, then the store: queries to q_out, keys and values to the cache.
//
//   x [tokens, ld] float32: a row holds nq = Gq * D query channels, nk = Gk * D key channels, nv = Hv * Dv value channels.
//   y_t[c] = sum_j cw[c][j] * u_(t - taps + 1 + j)[c], u before the sequence's start being zero. u of positions before
//   this step comes from the request's state, which holds the last taps - 1 projection rows: state[slot][i] is the row
//   of position starts - (taps - 1) + i. Positions of this step come from x itself (the step's rows are consecutive).
//   Norm: y / sqrt(mean(y^2) + eps) * w over each group, w [D] shared by all groups (nullptr: no norm).
//   Keys [pages, Gk, page_size, D]; values transposed within the page, [pages, Hv, Dv, page_size].
// A wave owns one unit of one token: a group of D query or key channels, or a head's Dv value channels (a lane holds
// up to CONV_PER of them, 64 apart); a block four units.
#define CONV_PER 16
template <typename T, typename TW>
__global__ __launch_bounds__(256) void conv_norm_store_kernel(
    const float* __restrict__ x, int ld, const TW* __restrict__ cw, int taps, const float* __restrict__ state,
    const int* __restrict__ state_slots, const int* __restrict__ token_row, const int* __restrict__ pos,
    const int* __restrict__ row_start, const int* __restrict__ starts, const TW* __restrict__ qw, const TW* __restrict__ kw,
    float eps, T* __restrict__ q_out, const int* __restrict__ slots, T* __restrict__ kc, T* __restrict__ vc, int Gq, int Gk,
    int Hv, int D, int Dv, int page_size) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int u = blockIdx.y * (256 / WAVE) + wave;
  if (u >= Gq + Gk + Hv) return;
  const int t = blockIdx.x, b = token_row[t], p = pos[t];
  const int start = starts[b], first = row_start[b];
  const int nq = Gq * D, nk = Gk * D, C = nq + nk + Hv * Dv;
  const bool is_q = u < Gq, is_v = u >= Gq + Gk;
  const int n = is_v ? Dv : D;
  const int cb = is_v ? nq + nk + (u - Gq - Gk) * Dv : u * D;  // the key groups follow the query groups
  const float* old = state + (size_t)state_slots[b] * (taps - 1) * C;
  float y[CONV_PER];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < CONV_PER; ++i) {
    const int d = lane + i * WAVE;
    y[i] = 0.f;
    if (d >= n) continue;
    const int c = cb + d;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int sp = p - taps + 1 + j;
      if (sp < 0) continue;
      const float v = sp >= start ? x[(size_t)(first + sp - start) * ld + c] : old[(size_t)(taps - 1 - (start - sp)) * C + c];
      acc = fmaf(to_f32(cw[(size_t)c * taps + j]), v, acc);
    }
    y[i] = acc;
    ss += acc * acc;
  }
  const int s = slots[t], page = s / page_size, off = s % page_size;
  if (is_v) {
    T* dst = vc + ((size_t)page * Hv + (u - Gq - Gk)) * Dv * page_size + off;
#pragma unroll
    for (int i = 0; i < CONV_PER; ++i) {
      const int e = lane + i * WAVE;
      if (e < n) dst[(size_t)e * page_size] = from_f32<T>(y[i]);
    }
    return;
  }
  const TW* w = is_q ? qw : kw;
  const float r = w ? 1.f / sqrtf(wave_sum(ss) / (float)D + eps) : 1.f;
  T* dst = is_q ? q_out + (size_t)t * nq + (size_t)u * D : kc + (((size_t)page * Gk + (u - Gq)) * page_size + off) * D;
#pragma unroll
  for (int i = 0; i < CONV_PER; ++i) {
    const int d = lane + i * WAVE;
    if (d < n) dst[d] = from_f32<T>(w ? y[i] * r * to_f32(w[d]) : y[i]);
  }
}

// After the step: the state takes the projection rows of the row's last taps - 1 positions. A thread owns one channel of
// one request and walks its taps - 1 entries upwards; an entry that stays (the step was shorter than the state) moves
// down from a higher index, which has not been written yet.
__global__ void conv_state_update_kernel(const float* __restrict__ x, int ld, int C, int taps, float* __restrict__ state,
                                         const int* __restrict__ state_slots, const int* __restrict__ row_start,
                                         const int* __restrict__ starts, int rows) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
  if (c >= C || b >= rows) return;
  const int first = row_start[b], n = row_start[b + 1] - first, start = starts[b];
  float* st = state + (size_t)state_slots[b] * (taps - 1) * C;
  for (int i = 0; i < taps - 1; ++i) {
    const int sp = start + n - (taps - 1) + i;
    float u = 0.f;
    if (sp >= start) u = x[(size_t)(first + sp - start) * ld + c];
    else if (sp >= 0) u = st[(size_t)(i + n) * C + c];
    st[(size_t)i * C + c] = u;
  }
}

extern "C" int ms_conv_norm_store(const float* x, int ld, const void* cw, int w_is_bf16, int taps, float* state,
                                  const int* state_slots, const int* token_row, const int* pos, const int* row_start,
                                  const int* starts, const void* qw, const void* kw, float eps, void* q_out, const int* slots,
                                  void* kc, void* vc, int out_is_bf16, int tokens, int rows, int Gq, int Gk, int Hv, int D, int Dv,
                                  int page_size, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  const long C = (long)(Gq + Gk) * D + (long)Hv * Dv;
  if (taps < 1 || Gq <= 0 || Gk <= 0 || Hv <= 0 || D <= 0 || Dv <= 0 || page_size <= 0 || ld < C || rows <= 0 || rows > 65535 ||
      !(eps >= 0.f) || (taps > 1 && state == nullptr) || slots == nullptr || (qw == nullptr) != (kw == nullptr))
    return MS_BAD_ARG;
  if (D > CONV_PER * WAVE || Dv > CONV_PER * WAVE) return MS_UNSUPPORTED;
  const int units = Gq + Gk + Hv;
  if ((units + 3) / 4 > 65535) return MS_BAD_ARG;
  const dim3 grid(tokens, (units + 3) / 4);
#define CV(T, TW)                                                                                                             \
  conv_norm_store_kernel<T, TW><<<grid, 256, 0, st>>>(x, ld, (const TW*)cw, taps, state, state_slots, token_row, pos, row_start, \
                                                      starts, (const TW*)qw, (const TW*)kw, eps, (T*)q_out, slots, (T*)kc, (T*)vc, \
                                                      Gq, Gk, Hv, D, Dv, page_size)
  if (out_is_bf16) {
    if (w_is_bf16) CV(bf16, bf16); else CV(bf16, float);
  } else {
    if (w_is_bf16) CV(float, bf16); else CV(float, float);
  }
#undef CV
  if (taps > 1)
    conv_state_update_kernel<<<dim3((unsigned)((C + 255) / 256), rows), 256, 0, st>>>(x, ld, (int)C, taps, state, state_slots,
                                                                                      row_start, starts, rows);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// Two score maps over the same values, combined per head: o = a1 - lambda * a2, divided by its root mean square over
// the head's E values (eps inside the root, no weight), times out_scale. `a` holds the maps' outputs as the attention
// kernel leaves them (float32, or the storage type), [tokens, G, 2, R, E]: key/value group, map, the group's R query heads. Output [tokens, G * R * E],
// head h = g * R + r. One block per token, a wave per head in turn.
template <typename T, typename TO>
__global__ __launch_bounds__(256) void map_difference_norm_kernel(const T* __restrict__ a, TO* __restrict__ out, int G, int R, int E,
                                                                  float lambda, float eps, float out_scale) {
  const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const T* row = a + (size_t)t * G * 2 * R * E;
  for (int h = wave; h < G * R; h += 256 / WAVE) {
    const int g = h / R, r = h % R;
    const T* a1 = row + ((size_t)(g * 2) * R + r) * E;
    const T* a2 = row + ((size_t)(g * 2 + 1) * R + r) * E;
    float ss = 0.f;
    for (int e = lane; e < E; e += WAVE) {
      const float o = to_f32(a1[e]) - lambda * to_f32(a2[e]);
      ss += o * o;
    }
    const float k = out_scale / sqrtf(wave_sum(ss) / (float)E + eps);
    TO* dst = out + ((size_t)t * G * R + h) * E;
    for (int e = lane; e < E; e += WAVE) dst[e] = from_f32<TO>((to_f32(a1[e]) - lambda * to_f32(a2[e])) * k);
  }
}

extern "C" int ms_map_difference_norm(const void* a, void* out, int in_is_bf16, int out_is_bf16, int tokens, int G, int R, int E,
                                      float lambda, float eps, float out_scale, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (G <= 0 || R <= 0 || E <= 0 || !(eps >= 0.f) || (in_is_bf16 && !out_is_bf16)) return MS_BAD_ARG;
  if (in_is_bf16) map_difference_norm_kernel<bf16, bf16><<<tokens, 256, 0, st>>>((const bf16*)a, (bf16*)out, G, R, E, lambda, eps, out_scale);
  else if (out_is_bf16) map_difference_norm_kernel<float, bf16><<<tokens, 256, 0, st>>>((const float*)a, (bf16*)out, G, R, E, lambda, eps, out_scale);
  else map_difference_norm_kernel<float, float><<<tokens, 256, 0, st>>>((const float*)a, (float*)out, G, R, E, lambda, eps, out_scale);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// Latent attention, before the attention kernel. A token's projection row x [ld] (float32) holds, from q_col on, H
// query heads of Dn plain and R rotated elements each, and, from kv_col on (kv_col < 0: this layer keeps nothing), C
// latent elements and R elements of the one key part that every head shares.
//   The first `rot` of the R elements are turned in pairs, (j, j + rot/2) or (2j, 2j + 1), by the angle whose cosine
//   and sine are rope[t][j] and rope[t][rot/2 + j]; the rest pass.
//   q_plain [tokens, H * Dn]: the plain query parts (a per-head matrix product takes them into the latent's space);
//   q_full [tokens, H * (C + R)]: only the turned parts are written here, behind each head's C columns;
//   cache row of the token's slot, [C + R]: the latent after its RMS norm (weight cw), then the turned key part;
//   the normed latent once more as the token's value, transposed within the page ([pages, C, page_size]): the tokens of
//   one element side by side, the order in which the matrix cores take the values.
// One block per token.
template <typename T, typename TW>
__global__ __launch_bounds__(256) void latent_prepare_kernel(const float* __restrict__ x, int ld, int q_col, int kv_col,
                                                             const float* __restrict__ rope, int rot, int pairing,
                                                             const TW* __restrict__ cw, float eps, T* __restrict__ q_plain,
                                                             T* __restrict__ q_full, const int* __restrict__ slots,
                                                             T* __restrict__ kc, T* __restrict__ vc, int page_size, int H, int Dn,
                                                             int R, int C) {
  __shared__ float red[256 / WAVE];
  const int t = blockIdx.x;
  const float* row = x + (size_t)t * ld;
  const float* cs = rot > 0 ? rope + (size_t)t * rot : nullptr;
  const int half = rot / 2;
  // element r of a turned part: its partner and the angle's index
  auto turned = [&](const float* v, int r) -> float {
    if (r >= rot) return v[r];
    int j, other;
    bool low;
    if (pairing == MS_ROPE_ADJACENT) {
      j = r / 2, low = (r % 2) == 0, other = low ? r + 1 : r - 1;
    } else {
      low = r < half, j = low ? r : r - half, other = low ? r + half : r - half;
    }
    const float c = cs[j], s = cs[half + j];
    return low ? v[r] * c - v[other] * s : v[r] * c + v[other] * s;
  };
  const float* qrow = row + q_col;
  for (int i = threadIdx.x; i < H * (Dn + R); i += 256) {
    const int h = i / (Dn + R), d = i % (Dn + R);
    if (d < Dn) q_plain[(size_t)t * H * Dn + (size_t)h * Dn + d] = from_f32<T>(qrow[i]);
    else q_full[(size_t)t * H * (C + R) + (size_t)h * (C + R) + C + (d - Dn)] = from_f32<T>(turned(qrow + (size_t)h * (Dn + R) + Dn, d - Dn));
  }
  if (kv_col < 0) return;
  const float* kv = row + kv_col;
  float ss = 0.f;
  for (int j = threadIdx.x; j < C; j += 256) ss += kv[j] * kv[j];
  const float r = 1.f / sqrtf(block_sum<256>(ss, red) / (float)C + eps);
  const int slot = slots[t], page = slot / page_size, off = slot % page_size;
  T* dst = kc + (size_t)slot * (C + R);
  T* val = vc + (size_t)page * C * page_size + off;
  for (int j = threadIdx.x; j < C; j += 256) {
    const T c = from_f32<T>(kv[j] * r * to_f32(cw[j]));
    dst[j] = c;
    val[(size_t)j * page_size] = c;
  }
  for (int j = threadIdx.x; j < R; j += 256) dst[C + j] = from_f32<T>(turned(kv + C, j));
}

extern "C" int ms_latent_prepare(const float* x, int ld, int q_col, int kv_col, const float* rope, int rot, int pairing,
                                 const void* cw, int w_is_bf16, float eps, void* q_plain, void* q_full, const int* slots,
                                 void* kc, void* vc, int page_size, int out_is_bf16, int tokens, int H, int Dn, int R, int C,
                                 hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (H <= 0 || Dn <= 0 || R < 0 || C <= 0 || rot < 0 || rot > R || rot % 2 || (rot > 0 && rope == nullptr) ||
      (pairing != MS_ROPE_HALVES && pairing != MS_ROPE_ADJACENT) || q_col < 0 || ld < q_col + H * (Dn + R) ||
      (kv_col >= 0 && (ld < kv_col + C + R || slots == nullptr || kc == nullptr || vc == nullptr || cw == nullptr || page_size < 1)) ||
      !(eps >= 0.f))
    return MS_BAD_ARG;
#define LP(T, TW)                                                                                                             \
  latent_prepare_kernel<T, TW><<<tokens, 256, 0, st>>>(x, ld, q_col, kv_col, rope, rot, pairing, (const TW*)cw, eps, (T*)q_plain, \
                                                       (T*)q_full, slots, (T*)kc, (T*)vc, page_size, H, Dn, R, C)
  if (out_is_bf16) {
    if (w_is_bf16) LP(bf16, bf16); else LP(bf16, float);
  } else {
    if (w_is_bf16) LP(float, bf16); else LP(float, float);
  }
#undef LP
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// A gate per head: o[t][h][:] *= sigmoid(x[t][col + h]), in place; x float32 with row stride ld, o [tokens, H * E].
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ o, const float* __restrict__ x, int ld, int col, int H, int E, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const size_t t = i / ((size_t)H * E);
  const int h = (int)((i / E) % H);
  const float g = 1.f / (1.f + expf(-x[t * ld + col + h]));
  o[i] = from_f32<T>(to_f32(o[i]) * g);
}

extern "C" int ms_head_gate(void* o, int is_bf16, const float* x, int ld, int col, int tokens, int H, int E, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (H <= 0 || E <= 0 || col < 0 || ld < col + H) return MS_BAD_ARG;
  const size_t n = (size_t)tokens * H * E;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (is_bf16) head_gate_kernel<bf16><<<blocks, 256, 0, st>>>((bf16*)o, x, ld, col, H, E, n);
  else head_gate_kernel<float><<<blocks, 256, 0, st>>>((float*)o, x, ld, col, H, E, n);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// out = act(x), elementwise: float32 in, float32 or bfloat16 out (the activation of a feed-forward without a gate).
template <typename T>
__global__ void activate_kernel(const float* __restrict__ x, T* __restrict__ out, size_t n, int act) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<T>(activate(x[i], act));
}

extern "C" int ms_activate(const float* x, void* out, int out_is_bf16, long long n, int act, hipStream_t st) {
  if (n <= 0) return MS_OK;
  if (!ms_act_ungated_ok(act)) return MS_BAD_ARG;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (out_is_bf16) activate_kernel<bf16><<<blocks, 256, 0, st>>>(x, (bf16*)out, (size_t)n, act);
  else activate_kernel<float><<<blocks, 256, 0, st>>>(x, (float*)out, (size_t)n, act);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// A matrix product per head in one launch, on the matrix cores: out[m][h * out_stride + col0 + n] = sum_k x[m][h * K + k] *
// w[h][n][k], x [M, ld >= H K] and w [H, N, K] bfloat16, float32 sums (v_mfma_f32_16x16x32_bf16), the result bfloat16 or
// float32. A block owns 64 rows x 64 columns of one head, a wave 16 of the rows; both operands come straight from
// memory, 16 bytes a lane (the weights of a head are small and stay in the cache). K a multiple of 8.
// gate (optional): float32 rows of stride gate_ld; head h's results of row m are multiplied by sigmoid(gate[m][gate_col + h]).
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 hg_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float hg_floatx4;

__device__ __forceinline__ hg_bf16x8 hg_load(const bf16* p, bool ok) {
  union { uint4 u; hg_bf16x8 v; } x;
  x.u = ok ? *reinterpret_cast<const uint4*>(p) : make_uint4(0, 0, 0, 0);
  return x.v;
}

__global__ __launch_bounds__(256) void head_gemm_bf16_kernel(const bf16* __restrict__ x, int ldx, const bf16* __restrict__ w,
                                                             void* __restrict__ out, int ldc, int out_stride, int col0, int M, int N,
                                                             int K, int out_f32, const float* __restrict__ gate, int gate_ld,
                                                             int gate_col) {
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, l16 = lane % 16, grp = lane / 16;
  const int h = blockIdx.z, m0 = blockIdx.x * 64 + wave * 16, n0 = blockIdx.y * 64;
  if (m0 >= M) return;
  const bool row_ok = m0 + l16 < M;
  const bf16* xp = x + (size_t)(m0 + l16) * ldx + (size_t)h * K + grp * 8;
  const bf16* wp[4];
  bool col_ok[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    col_ok[nt] = n0 + nt * 16 + l16 < N;
    wp[nt] = w + ((size_t)h * N + n0 + nt * 16 + l16) * K + grp * 8;
  }
  hg_floatx4 acc[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) acc[nt] = hg_floatx4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 64) {
    hg_bf16x8 a[2], b[2][4];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int k = k0 + c * 32;
      const bool in = k + grp * 8 < K;  // K is a multiple of 8: a lane's eight elements are all inside or all outside
      a[c] = hg_load(xp + k, in && row_ok);
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) b[c][nt] = hg_load(wp[nt] + k, in && col_ok[nt]);
    }
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[c], b[c][nt], acc[nt], 0, 0, 0);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int m = m0 + grp * 4 + r;
    if (m >= M) continue;
    const size_t at = (size_t)m * ldc + (size_t)h * out_stride + col0 + n0 + l16;
    const float gm = gate ? 1.f / (1.f + expf(-gate[(size_t)m * gate_ld + gate_col + h])) : 1.f;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      if (!col_ok[nt]) continue;
      if (out_f32) ((float*)out)[at + nt * 16] = acc[nt][r] * gm;
      else ((bf16*)out)[at + nt * 16] = static_cast<bf16>(acc[nt][r] * gm);
    }
  }
}

extern "C" int ms_head_gemm_bf16(const void* x, int ldx, const void* w, void* out, int ldc, int out_stride, int col0, int out_f32,
                                 int M, int H, int N, int K, const float* gate, int gate_ld, int gate_col, hipStream_t st) {
  if (M <= 0 || H <= 0 || N <= 0) return MS_OK;
  if (K <= 0 || ldx < H * K || out_stride < col0 + N || ldc < H * out_stride || col0 < 0 || H > 65535 || (N + 63) / 64 > 65535)
    return MS_BAD_ARG;
  if (gate && (gate_col < 0 || gate_ld < gate_col + H)) return MS_BAD_ARG;
  if (K % 8 || ldx % 8 || ((size_t)x % 16) || ((size_t)w % 16)) return MS_UNSUPPORTED;
  head_gemm_bf16_kernel<<<dim3((M + 63) / 64, (N + 63) / 64, H), 256, 0, st>>>((const bf16*)x, ldx, (const bf16*)w, out, ldc, out_stride,
                                                                             col0, M, N, K, out_f32, gate, gate_ld, gate_col);
  return launch_status();
}
