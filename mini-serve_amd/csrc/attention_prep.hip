// Between the fused q/k/v projection and the attention kernels, the form with every option a parameter: a rotation over
// part of a head in either pairing, an RMS norm per head before the rotation or behind it, with a weight or without,
// values of a width of their own, and values blended with another layer's values of the same token.
//
// qkv [tokens, ld >= Hq D + Hkv D + Hkv Dv] float32 (the projections' unrounded sums). One wave per (token, unit):
// units [0, Hq) are query heads, [Hq, Hq + Hkv) key heads, [Hq + Hkv, Hq + 2 Hkv) value heads.
//   q, k: norm_order MS_NORM_BEFORE: x <- x / rms(x) * w, then the rotation; MS_NORM_AFTER: the rotation, then
//         x <- x / rms(x) * w (a rotation whose cosines and sines carry a magnitude changes the head's length, so the two
//         differ); MS_NORM_NONE: the rotation alone. w == nullptr: no weight. The rotation turns pair j of the first `rot`
//         elements by the angle whose cosine and sine are rope[t][j] and rope[t][rot/2 + j].
//   v:    with v_first, v <- (1 - blend) v + blend v_first[t][h Dv + d] (float32 rows of stride v_first_ld).
//   q goes to q_out [tokens, Hq D]; k and v go to the cache page of the token's slot (slot = page * page_size + offset;
//   keys [pages, Hkv, page_size, D], values transposed within the page, [pages, Hkv, Dv, page_size]).
// With slots == nullptr only the query heads are processed. Everything is float32 until the one rounding of the store.
#include "common.h"

#define MS_NORM_NONE 0
#define MS_NORM_BEFORE 1
#define MS_NORM_AFTER 2
#define PREP_MAX_DIM 1024
#define PREP_PER_LANE (PREP_MAX_DIM / WAVE)

template <typename T, typename TW>
__global__ __launch_bounds__(256) void head_prepare_store_kernel(
    const float* __restrict__ qkv, int ld, T* __restrict__ q_out, const int* __restrict__ slots, const TW* __restrict__ qw,
    const TW* __restrict__ kw, int norm_order, float eps, const float* __restrict__ rope, int rot, int pairing,
    const float* __restrict__ v_first, int v_first_ld, float blend, T* __restrict__ kc, T* __restrict__ vc, int Hq, int Hkv,
    int D, int Dv, int page_size, int units) {
  const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int unit = blockIdx.y * 4 + wave;
  if (unit >= units) return;
  const float* row = qkv + (size_t)t * ld;
  const int s = slots ? slots[t] : 0;
  const size_t page = (size_t)(s / page_size), off = (size_t)(s % page_size);
  if (unit >= Hq + Hkv) {  // a value head
    const int h = unit - Hq - Hkv;
    const float* src = row + (size_t)Hq * D + (size_t)Hkv * D + (size_t)h * Dv;
    const float* first = v_first ? v_first + (size_t)t * v_first_ld + (size_t)h * Dv : nullptr;
    for (int d = lane; d < Dv; d += WAVE) {
      float v = src[d];
      if (first) v = (1.f - blend) * v + blend * first[d];
      vc[((page * Hkv + h) * Dv + d) * page_size + off] = from_f32<T>(v);
    }
    return;
  }
  const bool is_q = unit < Hq;
  const int h = is_q ? unit : unit - Hq;
  const float* src = row + (is_q ? (size_t)h * D : (size_t)Hq * D + (size_t)h * D);
  const TW* w = is_q ? qw : kw;
  const int half = rot / 2;
  const float* cs = rot > 0 ? rope + (size_t)t * rot : nullptr;
  float pre = 1.f;
  if (norm_order == MS_NORM_BEFORE) {
    float ss = 0.f;
    for (int d = lane; d < D; d += WAVE) ss += src[d] * src[d];
    pre = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
  }
  const bool w_before = norm_order == MS_NORM_BEFORE && w != nullptr;
  float vals[PREP_PER_LANE];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < PREP_PER_LANE; ++i) {
    const int d = lane + i * WAVE;
    float v = 0.f;
    if (d < D) {
      v = src[d] * pre * (w_before ? to_f32(w[d]) : 1.f);
      if (d < rot) {
        const bool adjacent = pairing == MS_ROPE_ADJACENT;
        const bool first = adjacent ? (d & 1) == 0 : d < half;
        const int j = adjacent ? d / 2 : (d < half ? d : d - half);
        const int pd = adjacent ? (d ^ 1) : (d < half ? d + half : d - half);
        const float p = src[pd] * pre * (w_before ? to_f32(w[pd]) : 1.f);
        v = first ? v * cs[j] - p * cs[half + j] : v * cs[j] + p * cs[half + j];
      }
    }
    vals[i] = v;
    ss += v * v;
  }
  float post = 1.f;
  if (norm_order == MS_NORM_AFTER) post = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
  const bool w_after = norm_order == MS_NORM_AFTER && w != nullptr;
#pragma unroll
  for (int i = 0; i < PREP_PER_LANE; ++i) {
    const int d = lane + i * WAVE;
    if (d >= D) continue;
    const float v = vals[i] * post * (w_after ? to_f32(w[d]) : 1.f);
    if (is_q) q_out[(size_t)t * Hq * D + (size_t)h * D + d] = from_f32<T>(v);
    else kc[((page * Hkv + h) * page_size + off) * D + d] = from_f32<T>(v);
  }
}

extern "C" int ms_head_prepare_store(const float* qkv, int ld, void* q_out, int is_bf16, const int* slots, const void* qw,
                                     const void* kw, int w_is_bf16, int norm_order, float eps, const float* rope, int rot,
                                     int pairing, const float* v_first, int v_first_ld, float blend, void* kc, void* vc,
                                     int tokens, int Hq, int Hkv, int D, int Dv, int page_size, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (qkv == nullptr || q_out == nullptr || Hq <= 0 || Hkv <= 0 || D <= 0 || Dv <= 0 || page_size <= 0 || rot < 0 || rot > D ||
      rot % 2 || (rot > 0) != (rope != nullptr) || ld < Hq * D + (slots ? Hkv * (D + Dv) : 0) ||
      (slots != nullptr && (kc == nullptr || vc == nullptr)) || !(eps >= 0.f) || tokens > 65535 * 32767 ||
      (v_first != nullptr && v_first_ld < Hkv * Dv))
    return MS_BAD_ARG;
  if (norm_order != MS_NORM_NONE && norm_order != MS_NORM_BEFORE && norm_order != MS_NORM_AFTER) return MS_BAD_ARG;
  if (norm_order == MS_NORM_NONE && (qw != nullptr || kw != nullptr)) return MS_BAD_ARG;
  if ((qw == nullptr) != (kw == nullptr)) return MS_BAD_ARG;
  if (D > PREP_MAX_DIM || Dv > PREP_MAX_DIM) return MS_UNSUPPORTED;
  if (rot > 0 && pairing != MS_ROPE_HALVES && pairing != MS_ROPE_ADJACENT) return MS_UNSUPPORTED;
  const int units = slots ? Hq + 2 * Hkv : Hq;
  if ((units + 3) / 4 > 65535) return MS_BAD_ARG;
  const dim3 grid(tokens, (units + 3) / 4);
#define PREP(T, TW) head_prepare_store_kernel<T, TW><<<grid, 256, 0, st>>>(qkv, ld, (T*)q_out, slots, (const TW*)qw, (const TW*)kw, norm_order, eps, rope, rot, pairing, v_first, v_first_ld, blend, (T*)kc, (T*)vc, Hq, Hkv, D, Dv, page_size, units)
  if (is_bf16) { if (w_is_bf16) PREP(bf16, bf16); else PREP(bf16, float); }
  else { if (w_is_bf16) PREP(float, bf16); else PREP(float, float); }
#undef PREP
  return launch_status();
}
