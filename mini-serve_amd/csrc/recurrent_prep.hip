// What recurrent mixers do to their projections before the recurrence runs, all in float32:
//   * a rotation of the query and key heads of a float32 projection, in place, with a scale on the way;
//   * the blends of a token's input with the previous token's, one per projection, and the carry of the last input;
//   * the last step of a decay per channel and token out of a small two-step projection.
#include "common.h"

// ---------------------------------------------------------------------------------------------
// x[t, col + h D + d] for h < H, d < D, in place: the first `rot` elements of each head are turned in pairs (j, j + rot/2)
// (or (2j, 2j + 1)) by the angles of rope[t] (cosines, then sines), then every element of the head is multiplied by
// `scale`. A thread owns a pair, or one element behind the rotated part: nothing is read by one thread and written by
// another. One block per token.
__global__ __launch_bounds__(256) void rotate_columns_kernel(float* __restrict__ x, int ld, int col, int H, int D,
                                                             const float* __restrict__ rope, int rot, int pairing, float scale) {
  const int t = blockIdx.x;
  float* row = x + (size_t)t * ld + col;
  const int half = rot / 2;
  const int per = D - half;  // items of a head: rot / 2 pairs and D - rot single elements
  const float* cs = rot > 0 ? rope + (size_t)t * rot : nullptr;
  for (int item = threadIdx.x; item < H * per; item += 256) {
    const int h = item / per, i = item % per;
    float* hd = row + h * D;
    if (i < half) {
      const int a = pairing == MS_ROPE_ADJACENT ? 2 * i : i;
      const int b = pairing == MS_ROPE_ADJACENT ? 2 * i + 1 : i + half;
      const float u = hd[a], v = hd[b];
      const float c = cs[i], s = cs[half + i];
      hd[a] = (u * c - v * s) * scale;
      hd[b] = (v * c + u * s) * scale;
    } else {
      hd[i + half] *= scale;  // element rot + (i - rot / 2)
    }
  }
}

extern "C" int ms_rotate_columns(float* x, int ld, int col, int tokens, int H, int D, const float* rope, int rot, int pairing,
                                 float scale, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (x == nullptr || H <= 0 || D <= 0 || col < 0 || col + H * D > ld || rot < 0 || rot > D || rot % 2 || (rot > 0 && rope == nullptr))
    return MS_BAD_ARG;
  if (pairing != MS_ROPE_HALVES && pairing != MS_ROPE_ADJACENT) return MS_UNSUPPORTED;
  rotate_columns_kernel<<<tokens, 256, 0, st>>>(x, ld, col, H, D, rope, rot, pairing, scale);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// out[s][t][c] = h[t][c] + (prev[t][c] - h[t][c]) * mu[s][c] for s < n: prev is the row before t in the step when t is not
// the first token of its request's rows, else the request's carried row carry[slot] (zeros when the request starts in this
// step). Float32 arithmetic, rounded once. The thread that reads carry[slot][c] for a request's first token is the one that
// then writes the request's last row of this step there: one reader and one writer per element, the same thread.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(const T* __restrict__ h, const T* __restrict__ mu, T* __restrict__ out,
                                                              float* __restrict__ carry, const int* __restrict__ token_row,
                                                              const int* __restrict__ row_start, const int* __restrict__ starts,
                                                              const int* __restrict__ state_slots, int tokens, int W, int n) {
  const int t = blockIdx.x;
  const int row = token_row[t];
  const int t0 = row_start[row], t1 = row_start[row + 1];
  const bool first = t == t0;
  const bool fresh = starts[row] == 0;
  float* cr = carry + (size_t)state_slots[row] * W;
  const T* hr = h + (size_t)t * W;
  const T* pr = first ? nullptr : h + (size_t)(t - 1) * W;
  const T* last = h + (size_t)(t1 - 1) * W;
  // a block per token and run of 256 VEC channels (few tokens still make many blocks); a thread owns VEC consecutive
  // channels, 16 bytes of a row (VEC = 1: any width)
  const int c0 = (blockIdx.y * 256 + threadIdx.x) * VEC;
  if (c0 >= W) return;
  struct alignas(sizeof(T) * VEC) Pack { T e[VEC]; };
  const Pack xs = *reinterpret_cast<const Pack*>(hr + c0);
  Pack ps, ls;
  if (!first) ps = *reinterpret_cast<const Pack*>(pr + c0);
  if (first) ls = *reinterpret_cast<const Pack*>(last + c0);
  float x[VEC], back[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    x[i] = to_f32(xs.e[i]);
    const float p = first ? (fresh ? 0.f : cr[c0 + i]) : to_f32(ps.e[i]);
    back[i] = p - x[i];
  }
  for (int s = 0; s < n; ++s) {
    const Pack ms = *reinterpret_cast<const Pack*>(mu + (size_t)s * W + c0);
    Pack o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) o.e[i] = from_f32<T>(x[i] + back[i] * to_f32(ms.e[i]));
    *reinterpret_cast<Pack*>(out + ((size_t)s * tokens + t) * W + c0) = o;
  }
  if (first)
#pragma unroll
    for (int i = 0; i < VEC; ++i) cr[c0 + i] = to_f32(ls.e[i]);
}

extern "C" int ms_token_shift_mix(const void* h, const void* mu, void* out, int is_bf16, float* carry, const int* token_row,
                                  const int* row_start, const int* starts, const int* state_slots, int tokens, int W, int n,
                                  hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (h == nullptr || mu == nullptr || out == nullptr || carry == nullptr || token_row == nullptr || row_start == nullptr ||
      starts == nullptr || state_slots == nullptr || W <= 0 || n <= 0)
    return MS_BAD_ARG;
  const int vec = is_bf16 ? 8 : 4;
  const bool wide = W % vec == 0 && (size_t)h % 16 == 0 && (size_t)mu % 16 == 0 && (size_t)out % 16 == 0;
  const int per = wide ? vec : 1;
  const dim3 grid(tokens, (W + 256 * per - 1) / (256 * per));
  if (grid.y > 65535) return MS_UNSUPPORTED;
#define TSM(T, V) token_shift_mix_kernel<T, V><<<grid, 256, 0, st>>>((const T*)h, (const T*)mu, (T*)out, carry, token_row, row_start, starts, state_slots, tokens, W, n)
  if (is_bf16) { if (wide) TSM(bf16, 8); else TSM(bf16, 1); }
  else { if (wide) TSM(float, 4); else TSM(float, 1); }
#undef TSM
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// z[t][c] <- -exp(z[t][c] + b[c]), or, as_decay, exp of that: the last step of a decay per channel and token,
// w = exp(-exp(W2 tanh(W1 x) + w0)). The two products and the tanh between them are the engine's float32 product and
// activation kernels; the logarithm -exp(...) is what the recurrence kernels take (a sum over tokens keeps it sharp where
// the decay is next to one). Float32, in place.
template <typename TB>
__global__ void neg_exp_bias_kernel(float* __restrict__ z, const TB* __restrict__ b, size_t n, int C, int as_decay) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  // (not below -200: the decay is zero in float32 from -104 on, and sums of such logarithms over a chunk of tokens keep
  // differences that are sharp in double precision)
  const float l = fmaxf(-expf(z[i] + to_f32(b[i % C])), -200.f);
  z[i] = as_decay ? expf(l) : l;
}

extern "C" int ms_neg_exp_bias(float* z, const void* b, int b_is_bf16, int tokens, int C, int as_decay, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (z == nullptr || b == nullptr || C <= 0) return MS_BAD_ARG;
  const size_t n = (size_t)tokens * C;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (b_is_bf16) neg_exp_bias_kernel<bf16><<<blocks, 256, 0, st>>>(z, (const bf16*)b, n, C, as_decay);
  else neg_exp_bias_kernel<float><<<blocks, 256, 0, st>>>(z, (const float*)b, n, C, as_decay);
  return launch_status();
}
