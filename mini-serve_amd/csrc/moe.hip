// A mixture of feed-forward experts (gated, act(gate x) * up x, or plain, act(up x)): routing, a plan that sorts the step's
// (token, chosen expert) pairs by expert, the two products per expert over the sorted pairs, and the weighted sum back
// into the stream. Router outputs from `real` on are identity experts: they have no weights, their pairs are left out of
// the plan, and the weighted sum adds the token's own input for them.
//
// A step of T tokens that each choose `top` of E experts has P = T top pairs; pair p = t * top + j is token t's j-th
// choice (largest logit first). The plan cuts every expert's run of pairs into tiles of `tile_rows` pairs; the product
// kernels are launched over the most tiles a step can have (ceil(P / tile_rows) + min(E, P)) and a block whose tile
// holds no pair leaves at once: nothing is read back to the host, and a captured step replays.
//
// A pair's result depends on its own row and its expert's weights alone (every output element is one dot product, summed
// in an order that its place in a tile does not change), so neither the order of the pairs inside an expert's run nor
// which other pairs the step holds changes a token's result; how many pairs it holds picks the size of the tiles, and
// the kernels of different tile sizes add in different orders (rounding of float32 sums). The sum over a token's choices
// runs in the order of the choices.
#include "common.h"

#define MOE_MAX_EXPERTS 512
#define MOE_MAX_TOP WAVE

// ---------------------------------------------------------------------------------------------
// Routing: z = logits[t] + bias; the `top` largest z (ties: the lower index), largest first; weights = softmax over
// those alone. One wave per token. The logits may come as `splits` partial sums `stride` floats apart (the router's
// product over few rows leaves them so), added here in ascending order.
template <typename TB>
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int ld, int splits, size_t stride,
                                                        const TB* __restrict__ bias, int T, int E, int top,
                                                        int* __restrict__ ids, float* __restrict__ weights) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  float z[MOE_MAX_EXPERTS / WAVE];
#pragma unroll
  for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i) {
    const int e = lane + i * WAVE;
    z[i] = e < E ? sum_splits(logits + (size_t)t * ld + e, splits, stride) + (bias ? to_f32(bias[e]) : 0.f) : -INFINITY;
  }
  float chosen = 0.f;  // lane j keeps the j-th chosen logit
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i)
      if (z[i] > best) { best = z[i]; at = lane + i * WAVE; }  // taken and absent experts hold -inf
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, WAVE);
      const int oa = __shfl_xor(at, off, WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (at >= E) at = j;  // logits that are no numbers: nothing to choose by, but the plan needs an expert that exists
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i)
      if (lane + i * WAVE == at) z[i] = -INFINITY;
    if (lane == 0) ids[(size_t)t * top + j] = at;
    if (lane == j) chosen = best;
  }
  // every chosen logit is at most the first; the sum runs in the order of the choices
  const float m = __shfl(chosen, 0, WAVE);
  float sum = 0.f;
  for (int j = 0; j < top; ++j) sum += expf(__shfl(chosen, j, WAVE) - m);
  if (lane < top) weights[(size_t)t * top + lane] = expf(chosen - m) / sum;
}

extern "C" int ms_moe_route(const float* logits, int ld, int splits, long long stride, const void* bias, int bias_is_bf16, int T,
                            int E, int top, int* ids, float* weights, hipStream_t st) {
  if (T <= 0) return MS_OK;
  if (logits == nullptr || ids == nullptr || weights == nullptr || E < 1 || top < 1 || top > E || ld < E || splits < 1 ||
      (splits > 1 && stride < (long long)T * ld))
    return MS_BAD_ARG;
  if (E > MOE_MAX_EXPERTS || top > MOE_MAX_TOP) return MS_UNSUPPORTED;
  const unsigned blocks = (unsigned)((T + 3) / 4);
  if (bias_is_bf16) moe_route_kernel<bf16><<<blocks, 256, 0, st>>>(logits, ld, splits, (size_t)stride, (const bf16*)bias, T, E, top, ids, weights);
  else moe_route_kernel<float><<<blocks, 256, 0, st>>>(logits, ld, splits, (size_t)stride, (const float*)bias, T, E, top, ids, weights);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// Routing by scores: s = softmax(logits[t]) over all E outputs; the choice is made by c = s + correction (correction may
// be absent), the weights are the chosen outputs' s as they stand (not renormalised). With groups > 1 the E outputs form
// `groups` equal groups of neighbours, a group's score is its largest c, and only outputs of the `keep` best groups
// (ties: the lower group) can be chosen: the others' c counts as minus infinity. The `top` largest c are chosen, largest
// first (ties: the lower index). One wave per token; s and c of a token pass through the wave's own rows of LDS.
template <typename TB>
__global__ __launch_bounds__(256) void moe_route_scored_kernel(const float* __restrict__ logits, int ld, int splits, size_t stride,
                                                               const TB* __restrict__ correction, int T, int E, int top,
                                                               int groups, int keep, int* __restrict__ ids,
                                                               float* __restrict__ weights) {
  __shared__ float ss[4][MOE_MAX_EXPERTS], cs[4][MOE_MAX_EXPERTS];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int t = blockIdx.x * 4 + wave;
  const bool live = t < T;  // every wave stays for the block's barriers
  float c[MOE_MAX_EXPERTS / WAVE];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i) {
    const int e = lane + i * WAVE;
    c[i] = (live && e < E) ? sum_splits(logits + (size_t)t * ld + e, splits, stride) : -INFINITY;
    m = fmaxf(m, c[i]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i) {
    c[i] = lane + i * WAVE < E ? expf(c[i] - m) : 0.f;
    sum += c[i];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i) {
    const int e = lane + i * WAVE;
    if (e < E) {
      const float sc = c[i] / sum;
      ss[wave][e] = sc;
      c[i] = sc + (correction ? to_f32(correction[e]) : 0.f);
      cs[wave][e] = c[i];
    } else {
      c[i] = -INFINITY;
    }
  }
  if (groups > 1) {
    const int n = E / groups;
    __syncthreads();
    float gm[MOE_MAX_EXPERTS / WAVE];  // lane l holds the scores of groups l, l + 64, ...
    bool taken[MOE_MAX_EXPERTS / WAVE];
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i) {
      const int g = lane + i * WAVE;
      gm[i] = -INFINITY;
      taken[i] = false;
      if (g < groups)
        for (int k = 0; k < n; ++k) gm[i] = fmaxf(gm[i], cs[wave][g * n + k]);
    }
    __syncthreads();  // cs is read; from here on it says which groups stay (1) and which do not (0)
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i)
      if (lane + i * WAVE < groups) cs[wave][lane + i * WAVE] = 0.f;
    for (int j = 0; j < keep; ++j) {
      float best = -INFINITY;
      int at = 0x7fffffff;
#pragma unroll
      for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i)
        if (lane + i * WAVE < groups && !taken[i] && (at == 0x7fffffff || gm[i] > best)) { best = gm[i]; at = lane + i * WAVE; }
#pragma unroll
      for (int off = WAVE / 2; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off, WAVE);
        const int oa = __shfl_xor(at, off, WAVE);
        if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
      }
#pragma unroll
      for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i)
        if (lane + i * WAVE == at) { taken[i] = true; cs[wave][at] = 1.f; }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i) {
      const int e = lane + i * WAVE;
      if (e < E && cs[wave][e / n] == 0.f) c[i] = -INFINITY;
    }
  } else {
    __syncthreads();
  }
  if (!live) return;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i)
      if (c[i] > best) { best = c[i]; at = lane + i * WAVE; }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, WAVE);
      const int oa = __shfl_xor(at, off, WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (at >= E) at = j;  // nothing left to choose by (no numbers, or fewer outputs in the kept groups than choices)
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / WAVE; ++i)
      if (lane + i * WAVE == at) c[i] = -INFINITY;
    if (lane == 0) {
      ids[(size_t)t * top + j] = at;
      weights[(size_t)t * top + j] = ss[wave][at];
    }
  }
}

extern "C" int ms_moe_route_scored(const float* logits, int ld, int splits, long long stride, const void* correction,
                                   int correction_is_bf16, int T, int E, int top, int groups, int keep, int* ids, float* weights,
                                   hipStream_t st) {
  if (T <= 0) return MS_OK;
  if (logits == nullptr || ids == nullptr || weights == nullptr || E < 1 || top < 1 || top > E || ld < E || splits < 1 ||
      (splits > 1 && stride < (long long)T * ld) || groups < 1 || E % groups || keep < 1 || keep > groups)
    return MS_BAD_ARG;
  if (E > MOE_MAX_EXPERTS || top > MOE_MAX_TOP) return MS_UNSUPPORTED;
  const unsigned blocks = (unsigned)((T + 3) / 4);
  if (correction_is_bf16) moe_route_scored_kernel<bf16><<<blocks, 256, 0, st>>>(logits, ld, splits, (size_t)stride, (const bf16*)correction, T, E, top, groups, keep, ids, weights);
  else moe_route_scored_kernel<float><<<blocks, 256, 0, st>>>(logits, ld, splits, (size_t)stride, (const float*)correction, T, E, top, groups, keep, ids, weights);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// The plan, one block: counts per expert, every expert's run of `order` (order[i] = the pair at sorted place i), and the
// tiles: tile n covers places tile_start[n] .. tile_start[n] + tile_count[n] - 1 of expert tile_expert[n]. Tiles past the
// last get a count of zero. Pairs whose id is E or more (identity experts) are in no run and no tile.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ ids, int P, int E, int tile_rows, int max_tiles,
                                                        int* __restrict__ order, int* __restrict__ tile_expert,
                                                        int* __restrict__ tile_start, int* __restrict__ tile_count) {
  __shared__ int counts[MOE_MAX_EXPERTS], offsets[MOE_MAX_EXPERTS], cursor[MOE_MAX_EXPERTS], tile_base[MOE_MAX_EXPERTS];
  __shared__ int total_tiles;
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += 1024) { counts[e] = 0; cursor[e] = 0; }
  __syncthreads();
  for (int p = tid; p < P; p += 1024)
    if (ids[p] < E) atomicAdd(&counts[max(ids[p], 0)], 1);
  __syncthreads();
  if (tid == 0) {
    int off = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = off;
      tile_base[e] = nt;
      off += counts[e];
      nt += (counts[e] + tile_rows - 1) / tile_rows;
    }
    total_tiles = nt;
  }
  __syncthreads();
  for (int e = tid; e < E; e += 1024) {
    const int n = (counts[e] + tile_rows - 1) / tile_rows;
    for (int i = 0; i < n; ++i) {
      const int at = tile_base[e] + i;
      if (at >= max_tiles) break;
      tile_expert[at] = e;
      tile_start[at] = offsets[e] + i * tile_rows;
      tile_count[at] = min(tile_rows, counts[e] - i * tile_rows);
    }
  }
  for (int n = total_tiles + tid; n < max_tiles; n += 1024) {
    tile_expert[n] = 0;
    tile_start[n] = 0;
    tile_count[n] = 0;
  }
  for (int p = tid; p < P; p += 1024) {
    if (ids[p] >= E) continue;
    const int e = max(ids[p], 0);
    order[offsets[e] + atomicAdd(&cursor[e], 1)] = p;
  }
}

extern "C" int ms_moe_plan(const int* ids, int P, int E, int tile_rows, int max_tiles, int* order, int* tile_expert,
                           int* tile_start, int* tile_count, hipStream_t st) {
  if (P <= 0) return MS_OK;
  if (ids == nullptr || order == nullptr || tile_expert == nullptr || tile_start == nullptr || tile_count == nullptr || E < 1 ||
      tile_rows < 1 || max_tiles < (P + tile_rows - 1) / tile_rows + (E < P ? E : P))
    return MS_BAD_ARG;
  if (E > MOE_MAX_EXPERTS) return MS_UNSUPPORTED;
  moe_plan_kernel<<<1, 1024, 0, st>>>(ids, P, E, tile_rows, max_tiles, order, tile_expert, tile_start, tile_count);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// The experts' products on the matrix cores (bfloat16 operands, float32 sums, v_mfma_f32_16x16x32_bf16), operands
// straight from memory, 16 bytes a lane. A wave owns 16 pairs x 16 NT columns; a block's four waves split a tile of 64
// pairs by rows (NT = 4: 64 columns a block), a tile of 16 pairs by columns (64 NT columns a block: steps of few tokens,
// where every chosen expert has a tile of its own and its weights are streamed once; the fewer tiles the step can have,
// the narrower the waves' runs of columns, so that the chip still gets waves enough to stream with).
//   MODE 1 (gated): rows are x[token of the pair] (K = the model's width), two weights per expert, gate and up [E, N, K];
//          the result act(gate) * up goes to h[sorted place][N] in the compute type.
//   MODE 2 (plain first product): the same rows, one weight per expert; act(up) goes to h[sorted place][N].
//   MODE 0: rows are h[sorted place] (K = the experts' width), one weight per expert [E, N, K]; the result times the pair's
//          routing weight goes to y[pair][N] in float32.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 moe_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float moe_floatx4;

// Eight consecutive elements from p + k, those at or past K zero. ALIGNED: one 16-byte load (K, the row strides and the
// bases are multiples of 8 elements, so a lane's eight are all inside or all outside).
template <bool ALIGNED> __device__ __forceinline__ moe_bf16x8 moe_load(const bf16* p, int k, int K, bool ok) {
  union { uint4 u; moe_bf16x8 v; bf16 e[8]; } x;
  x.u = make_uint4(0, 0, 0, 0);
  if (ALIGNED) {
    if (ok && k < K) x.u = *reinterpret_cast<const uint4*>(p + k);
  } else if (ok) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (k + i < K) x.e[i] = p[k + i];
  }
  return x.v;
}

template <int MODE, bool ALIGNED, int NT, bool KSPLIT = false>
__global__ __launch_bounds__(256) void moe_gemm_bf16_kernel(
    const bf16* __restrict__ a, int lda, const bf16* __restrict__ w1, const bf16* __restrict__ w2, void* __restrict__ out,
    const int* __restrict__ order, const int* __restrict__ tile_expert, const int* __restrict__ tile_start,
    const int* __restrict__ tile_count, const float* __restrict__ pair_weight, int top, int N, int K, int tile_rows, int act) {
  constexpr bool GATED = MODE == 1, FIRST = MODE != 0;
  const int count = tile_count[blockIdx.x];
  if (count == 0) return;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, l16 = lane % 16, grp = lane / 16;
  const bool by_rows = tile_rows == 64;
  const int m0 = by_rows ? wave * 16 : 0;
  // KSPLIT (16-pair tiles): the block's four waves share its 16 NT columns and take a quarter of K each (a multiple of 64),
  // so that four times the waves stream a step's weights; their sums meet in LDS and are added in wave order.
  const int n0 = (by_rows || KSPLIT) ? blockIdx.y * (16 * NT) : (blockIdx.y * 4 + wave) * (16 * NT);
  if (m0 >= count || n0 >= N) return;
  const int k_quarter = ((K + 3) / 4 + 63) / 64 * 64;
  const int k_lo = KSPLIT ? min(K, wave * k_quarter) : 0;
  const int k_hi = KSPLIT ? min(K, k_lo + k_quarter) : K;
  const int e = tile_expert[blockIdx.x], start = tile_start[blockIdx.x];
  const bool row_ok = m0 + l16 < count;
  const int place = start + m0 + (row_ok ? l16 : 0);
  const bf16* ap = a + (size_t)(FIRST ? order[place] / top : place) * lda;
  const bf16* wp1[NT];
  const bf16* wp2[NT];
  bool col_ok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    col_ok[nt] = n0 + nt * 16 + l16 < N;
    const size_t at = ((size_t)e * N + (col_ok[nt] ? n0 + nt * 16 + l16 : 0)) * K;
    wp1[nt] = w1 + at;
    wp2[nt] = GATED ? w2 + at : nullptr;
  }
  moe_floatx4 acc1[NT], acc2[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc1[nt] = acc2[nt] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
  // 64 k a step: a lane takes 16 consecutive k of its rows (two loads of 16 bytes: a wave reads a whole 128-byte line
  // of every row) and multiplies them in two products. Both operands are cut the same way, so the sum is over
  // every k once; within a step the order of k is that of the lanes' runs.
#pragma unroll(4 / NT)
  for (int k0 = k_lo; k0 < k_hi; k0 += 64) {
    const int kk = k0 + grp * 16;  // the lane's sixteen elements of this step
    moe_bf16x8 av[2], b1[NT][2], b2[NT][2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      av[u] = moe_load<ALIGNED>(ap, kk + 8 * u, k_hi, row_ok);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        b1[nt][u] = moe_load<ALIGNED>(wp1[nt], kk + 8 * u, k_hi, col_ok[nt]);
        if (GATED) b2[nt][u] = moe_load<ALIGNED>(wp2[nt], kk + 8 * u, k_hi, col_ok[nt]);
      }
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        acc1[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[u], b1[nt][u], acc1[nt], 0, 0, 0);
        if (GATED) acc2[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[u], b2[nt][u], acc2[nt], 0, 0, 0);
      }
  }
  if constexpr (KSPLIT) {
    __shared__ float meet[3][GATED ? 2 * NT : NT][4][WAVE];
    if (wave > 0) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          meet[wave - 1][nt][r][lane] = acc1[nt][r];
          if (GATED) meet[wave - 1][NT + nt][r][lane] = acc2[nt][r];
        }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          acc1[nt][r] += meet[w][nt][r][lane];
          if (GATED) acc2[nt][r] += meet[w][NT + nt][r][lane];
        }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int m = m0 + grp * 4 + r;
    if (m >= count) continue;
    if (GATED) {
      bf16* o = (bf16*)out + (size_t)(start + m) * N + n0 + l16;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        if (col_ok[nt]) o[nt * 16] = static_cast<bf16>(gated_value(acc1[nt][r], acc2[nt][r], act, 0.f));
    } else if (FIRST) {
      bf16* o = (bf16*)out + (size_t)(start + m) * N + n0 + l16;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        if (col_ok[nt]) o[nt * 16] = static_cast<bf16>(activate(acc1[nt][r], act));
    } else {
      const int pair = order[start + m];
      const float pw = pair_weight[pair];
      float* o = (float*)out + (size_t)pair * N + n0 + l16;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        if (col_ok[nt]) o[nt * 16] = acc1[nt][r] * pw;
    }
  }
}

// The same two products for steps with many pairs per expert (K a multiple of 64, rows 16-byte aligned): tiles of BM pairs
// x 128 weight rows, K in slabs of 64 that go straight into LDS (global_load_lds, 16 bytes a lane) in a ring of two
// stages, one barrier per slab, two blocks per CU. A load instruction of a wave fills 1 KB of LDS in lane order, that is
// 8 tile rows of 128 bytes; the 16-byte chunk c of tile row R lands in slot c ^ ((R >> 1) & 7) of its row, so that a
// fragment read (16 rows, one chunk column) touches every bank once. The weight rows are the matrix instruction's first
// operand and the pairs its second: a lane ends up with four consecutive columns of one pair.
//   GATED: the tile's weight rows are blocks of 16 gate rows and 16 up rows in turn (64 columns of h a block), so that a
//          lane's fragments 2 i and 2 i + 1 are gate and up of the same four outputs.
// Pairs past the tile's count read the tile's last pair, weight rows past N the last row: their results are not stored.
// Every output element is one chain of products over k in ascending slabs, whatever the tile and the pair's place in it.
template <int N_> __device__ __forceinline__ void moe_wait_loads() {
  __builtin_amdgcn_s_waitcnt((N_ & 15) | ((N_ >> 4) << 14) | (7 << 4) | (15 << 8));  // vmcnt alone
}

template <int MODE, int BM, int WR, int WC>
__global__ __launch_bounds__(256, 2) void moe_gemm_bf16_lds_kernel(
    const bf16* __restrict__ a, int lda, const bf16* __restrict__ w1, const bf16* __restrict__ w2, void* __restrict__ out,
    const int* __restrict__ order, const int* __restrict__ tile_expert, const int* __restrict__ tile_start,
    const int* __restrict__ tile_count, const float* __restrict__ pair_weight, int top, int N, int K, int act) {
  constexpr bool GATED = MODE == 1, FIRST = MODE != 0;
  static_assert(WR * WC == 4, "four waves a block");
  constexpr int BN = 128, KS = 64, STAGES = 2;
  constexpr int WM = BM / WR, WN = BN / WC, FM = WM / 16, FN = WN / 16;
  constexpr int ROW_BYTES = KS * 2, CPR = 8, RPI = 8;
  constexpr int XI = BM / (4 * RPI), WI = BN / (4 * RPI);
  constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
  static_assert(!GATED || FN % 2 == 0, "gate and up fragments come in pairs");
  extern __shared__ __attribute__((aligned(1024))) unsigned char moe_lds[];
  const int tile = blockIdx.y;
  const int count = tile_count[tile];
  if (count == 0) return;
  const int e = tile_expert[tile], start = tile_start[tile];
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 16, g = lane / 16;
  const int n0 = blockIdx.x * (GATED ? BN / 2 : BN);  // first output column of the tile
  const int wm = (wave / WC) * WM, wn = (wave % WC) * WN;
  const int slabs = K / KS;

  const int lrow = lane / CPR, lslot = lane % CPR;
  const bf16* xsrc[XI];
  const bf16* wsrc[WI];
#pragma unroll
  for (int j = 0; j < XI; ++j) {
    const int R = (wave * XI + j) * RPI + lrow;
    const int place = start + min(R, count - 1);
    xsrc[j] = a + (size_t)(FIRST ? order[place] / top : place) * lda + ((lslot ^ ((R >> 1) & (CPR - 1))) * 8);
  }
#pragma unroll
  for (int j = 0; j < WI; ++j) {
    const int R = (wave * WI + j) * RPI + lrow;
    const int chunk = (lslot ^ ((R >> 1) & (CPR - 1))) * 8;
    if (GATED) {
      const int n = min(n0 + (R / 32) * 16 + R % 16, N - 1);
      wsrc[j] = (((R / 16) & 1) ? w2 : w1) + ((size_t)e * N + n) * K + chunk;
    } else {
      wsrc[j] = w1 + ((size_t)e * N + min(n0 + R, N - 1)) * K + chunk;
    }
  }
  auto issue = [&](int slab) __attribute__((always_inline)) {
    unsigned char* stage = moe_lds + (slab % STAGES) * STAGE_BYTES;
#pragma unroll
    for (int j = 0; j < XI; ++j)
      __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(xsrc[j] + (size_t)slab * KS),
                                       (void __attribute__((address_space(3)))*)(stage + (wave * XI + j) * 1024), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < WI; ++j)
      __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(wsrc[j] + (size_t)slab * KS),
                                       (void __attribute__((address_space(3)))*)(stage + BM * ROW_BYTES + (wave * WI + j) * 1024),
                                       16, 0, 0);
  };

  moe_floatx4 acc[FN][FM];
#pragma unroll
  for (int i = 0; i < FN; ++i)
#pragma unroll
    for (int j = 0; j < FM; ++j) acc[i][j] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
  const int sw = (r >> 1) & (CPR - 1);
  const int x_off = (wm + r) * ROW_BYTES, w_off = BM * ROW_BYTES + (wn + r) * ROW_BYTES;

  issue(0);
  for (int k = 0; k < slabs; ++k) {
    moe_wait_loads<0>();
    __syncthreads();  // slab k has landed for every wave, and every wave is done with slab k - 1
    if (k + 1 < slabs) issue(k + 1);
    const unsigned char* stage = moe_lds + (k % STAGES) * STAGE_BYTES;
    moe_bf16x8 wf[2][FN], xf[2][FM];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int slot = ((t * 4 + g) ^ sw) * 16;
#pragma unroll
      for (int i = 0; i < FN; ++i) wf[t][i] = *reinterpret_cast<const moe_bf16x8*>(stage + w_off + i * 16 * ROW_BYTES + slot);
#pragma unroll
      for (int j = 0; j < FM; ++j) xf[t][j] = *reinterpret_cast<const moe_bf16x8*>(stage + x_off + j * 16 * ROW_BYTES + slot);
    }
    __builtin_amdgcn_sched_barrier(0);
    // an expert's last tile is seldom full: runs of 16 pairs past its count are not multiplied (the same for a whole wave)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < FM; ++j) {
        if (wm + j * 16 >= count) continue;
#pragma unroll
        for (int i = 0; i < FN; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[t][i], xf[t][j], acc[i][j], 0, 0, 0);
      }
  }

  const bool vec = N % 4 == 0;
#pragma unroll
  for (int j = 0; j < FM; ++j) {
    const int m = wm + j * 16 + r;
    if (m >= count) continue;
    if (GATED) {
      bf16* o = (bf16*)out + (size_t)(start + m) * N;
#pragma unroll
      for (int i = 0; i + 1 < FN; i += 2) {
        const int col = n0 + wn / 2 + (i / 2) * 16 + g * 4;
        union { uint2 u; bf16 v[4]; } q;
#pragma unroll
        for (int c = 0; c < 4; ++c) q.v[c] = static_cast<bf16>(gated_value(acc[i][j][c], acc[i + 1][j][c], act, 0.f));
        if (vec && col + 3 < N) *reinterpret_cast<uint2*>(o + col) = q.u;
        else
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (col + c < N) o[col + c] = q.v[c];
      }
    } else if (FIRST) {
      bf16* o = (bf16*)out + (size_t)(start + m) * N;
#pragma unroll
      for (int i = 0; i < FN; ++i) {
        const int col = n0 + wn + i * 16 + g * 4;
        union { uint2 u; bf16 v[4]; } q;
#pragma unroll
        for (int c = 0; c < 4; ++c) q.v[c] = static_cast<bf16>(activate(acc[i][j][c], act));
        if (vec && col + 3 < N) *reinterpret_cast<uint2*>(o + col) = q.u;
        else
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (col + c < N) o[col + c] = q.v[c];
      }
    } else {
      const int pair = order[start + m];
      const float pw = pair_weight[pair];
      float* o = (float*)out + (size_t)pair * N;
#pragma unroll
      for (int i = 0; i < FN; ++i) {
        const int col = n0 + wn + i * 16 + g * 4;
        if (vec && col + 3 < N) *reinterpret_cast<float4*>(o + col) = make_float4(acc[i][j][0] * pw, acc[i][j][1] * pw, acc[i][j][2] * pw, acc[i][j][3] * pw);
        else
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (col + c < N) o[col + c] = acc[i][j][c] * pw;
      }
    }
  }
}

template <int MODE, int BM, int WR, int WC>
static int moe_launch_lds(const void* a, int lda, const void* w1, const void* w2, void* out, const int* order, const int* tile_expert,
                          const int* tile_start, const int* tile_count, const float* pair_weight, int max_tiles, int top, int N,
                          int K, int act, hipStream_t st) {
  constexpr int lds_bytes = 2 * (BM + 128) * 128;
  static bool ready = false;  // more than 48 KB of LDS is asked for once per kernel
  if (!ready) {
    if (hipFuncSetAttribute((const void*)moe_gemm_bf16_lds_kernel<MODE, BM, WR, WC>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            lds_bytes) != hipSuccess)
      return MS_LAUNCH_FAILED;
    ready = true;
  }
  const int cols = MODE == 1 ? 64 : 128;
  const dim3 grid((N + cols - 1) / cols, max_tiles);
  if (grid.y > 65535) return MS_BAD_ARG;
  moe_gemm_bf16_lds_kernel<MODE, BM, WR, WC><<<grid, 256, lds_bytes, st>>>((const bf16*)a, lda, (const bf16*)w1, (const bf16*)w2, out, order,
                                                                           tile_expert, tile_start, tile_count, pair_weight, top, N, K, act);
  return launch_status();
}

// The same two products in true float32 on the vector units: 64 x 64 tiles through LDS, every output element one chain of
// fused multiply-adds over k in ascending order.
template <int MODE>
__global__ __launch_bounds__(256) void moe_gemm_f32_kernel(
    const float* __restrict__ a, int lda, const float* __restrict__ w1, const float* __restrict__ w2, float* __restrict__ out,
    const int* __restrict__ order, const int* __restrict__ tile_expert, const int* __restrict__ tile_start,
    const int* __restrict__ tile_count, const float* __restrict__ pair_weight, int top, int N, int K, int act) {
  constexpr bool GATED = MODE == 1, FIRST = MODE != 0;
  const int count = tile_count[blockIdx.x];
  if (count == 0) return;
  __shared__ float As[16][64 + 4];
  __shared__ float W1s[16][64 + 4];
  __shared__ float W2s[GATED ? 16 : 1][64 + 4];
  const int tid = threadIdx.x;
  const int e = tile_expert[blockIdx.x], start = tile_start[blockIdx.x];
  const int n0 = blockIdx.y * 64;
  const int tx = tid % 16, ty = tid / 16;      // 16 x 16 threads, 4 x 4 outputs each
  const int lr = tid / 4, lk = (tid % 4) * 4;  // loader: row within the tile, k offset
  const bool a_ok = lr < count;
  const float* arow = a + (size_t)(a_ok ? (FIRST ? order[start + lr] / top : start + lr) : 0) * lda;
  const bool w_ok = n0 + lr < N;
  const size_t wat = ((size_t)e * N + (w_ok ? n0 + lr : 0)) * K;
  float acc1[4][4], acc2[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc1[i][j] = acc2[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += 16) {
    float av[4], wv1[4], wv2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      av[i] = (a_ok && k < K) ? arow[k] : 0.f;
      wv1[i] = (w_ok && k < K) ? w1[wat + k] : 0.f;
      wv2[i] = (GATED && w_ok && k < K) ? w2[wat + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[lk + i][lr] = av[i];
      W1s[lk + i][lr] = wv1[i];
      if (GATED) W2s[lk + i][lr] = wv2[i];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      float x[4], u[4], v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u[j] = W1s[k][tx * 4 + j];
        v[j] = GATED ? W2s[k][tx * 4 + j] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc1[i][j] = fmaf(x[i], u[j], acc1[i][j]);
          if (GATED) acc2[i][j] = fmaf(x[i], v[j], acc2[i][j]);
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = ty * 4 + i;
    if (m >= count) continue;
    const int pair = FIRST ? 0 : order[start + m];
    const float pw = FIRST ? 1.f : pair_weight[pair];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      if (GATED) out[(size_t)(start + m) * N + n] = gated_value(acc1[i][j], acc2[i][j], act, 0.f);
      else if (FIRST) out[(size_t)(start + m) * N + n] = activate(acc1[i][j], act);
      else out[(size_t)pair * N + n] = acc1[i][j] * pw;
    }
  }
}

// a: the rows ([tokens, lda] for a first product, [P, lda] sorted places for the second); w1 (and w2, gated): [E, N, K];
// out: h [P, N] (a first product, the compute type) or y [P, N] float32. mode: 0 the second product, 1 the gated first
// product, 2 the plain first product. tile_rows: 16, 64 or 128 in bfloat16 (128: K a multiple of 64 and 16-byte aligned
// rows), 64 in float32.
extern "C" int ms_moe_gemm(const void* a, int lda, const void* w1, const void* w2, void* out, int is_bf16, int mode,
                           const int* order, const int* tile_expert, const int* tile_start, const int* tile_count,
                           const float* pair_weight, int max_tiles, int top, int N, int K, int tile_rows, int act, hipStream_t st) {
  if (max_tiles <= 0 || N <= 0) return MS_OK;
  const bool gated = mode == 1;
  if (mode < 0 || mode > 2 || a == nullptr || w1 == nullptr || (gated && w2 == nullptr) || out == nullptr || order == nullptr ||
      tile_expert == nullptr || tile_start == nullptr || tile_count == nullptr || (mode == 0 && pair_weight == nullptr) || top < 1 ||
      K <= 0 || lda < K || (gated && (act < 0 || act >= MS_ACT_COUNT)) || (mode == 2 && !ms_act_ungated_ok(act)))
    return MS_BAD_ARG;
  if (is_bf16) {
    if (tile_rows != 16 && tile_rows != 64 && tile_rows != 128) return MS_BAD_ARG;
    const bool rows16 = (size_t)a % 16 == 0 && (size_t)w1 % 16 == 0 && (!gated || (size_t)w2 % 16 == 0) && lda % 8 == 0;
    if (tile_rows >= 64 && K % 64 == 0 && rows16 && (mode != 0 || (size_t)out % 16 == 0)) {
#define MOE_LDS(G, BM, WR, WC) moe_launch_lds<G, BM, WR, WC>(a, lda, w1, w2, out, order, tile_expert, tile_start, tile_count, pair_weight, max_tiles, top, N, K, act, st)
      if (tile_rows == 128) return mode == 1 ? MOE_LDS(1, 128, 2, 2) : (mode == 2 ? MOE_LDS(2, 128, 2, 2) : MOE_LDS(0, 128, 2, 2));
      return mode == 1 ? MOE_LDS(1, 64, 1, 4) : (mode == 2 ? MOE_LDS(2, 64, 1, 4) : MOE_LDS(0, 64, 1, 4));
#undef MOE_LDS
    }
    if (tile_rows == 128) return MS_UNSUPPORTED;  // the caller plans tiles of 128 only where the kernel above takes them
    // 16-pair tiles: min(E, pairs) of them at most are in use, each times the column blocks; the narrowest run of columns
    // with which that is under four blocks a CU.
    int nt = 4;
    if (tile_rows == 16) {
      const long busy = max_tiles / 2 + 1;  // about half of the launched tiles hold pairs
      while (nt > 1 && busy * ((N + 64 * nt - 1) / (64 * nt)) < 1024) nt /= 2;
    }
    const bool aligned = K % 8 == 0 && lda % 8 == 0 && (size_t)a % 16 == 0 && (size_t)w1 % 16 == 0 && (!gated || (size_t)w2 % 16 == 0);
#define MOE_ARGS (const bf16*)a, lda, (const bf16*)w1, (const bf16*)w2, out, order, tile_expert, tile_start, tile_count, pair_weight, top, N, K, tile_rows, act
    // still few blocks at the narrowest columns: the waves of a block share 16 columns and split K
    if (tile_rows == 16 && nt == 1 && aligned && K >= 512 && (max_tiles / 2 + 1) * ((N + 63) / 64) < 2048 && (N + 15) / 16 <= 65535) {
      const dim3 grid(max_tiles, (N + 15) / 16);
      if (mode == 1) moe_gemm_bf16_kernel<1, true, 1, true><<<grid, 256, 0, st>>>(MOE_ARGS);
      else if (mode == 2) moe_gemm_bf16_kernel<2, true, 1, true><<<grid, 256, 0, st>>>(MOE_ARGS);
      else moe_gemm_bf16_kernel<0, true, 1, true><<<grid, 256, 0, st>>>(MOE_ARGS);
      return launch_status();
    }
    const int cols = tile_rows == 64 ? 64 : 64 * nt;
    const dim3 grid(max_tiles, (N + cols - 1) / cols);
    if (grid.y > 65535) return MS_BAD_ARG;
#define MOE(G, A, T) moe_gemm_bf16_kernel<G, A, T><<<grid, 256, 0, st>>>(MOE_ARGS)
#define MOE_NT(G, A) do { if (nt == 4) MOE(G, A, 4); else if (nt == 2) MOE(G, A, 2); else MOE(G, A, 1); } while (0)
#define MOE_AL(G) do { if (aligned) MOE_NT(G, true); else MOE_NT(G, false); } while (0)
    if (mode == 1) MOE_AL(1);
    else if (mode == 2) MOE_AL(2);
    else MOE_AL(0);
#undef MOE_AL
#undef MOE_NT
#undef MOE
#undef MOE_ARGS
  } else {
    if (tile_rows != 64) return MS_BAD_ARG;
    const dim3 grid(max_tiles, (N + 63) / 64);
    if (grid.y > 65535) return MS_BAD_ARG;
#define MOE_F32(G) moe_gemm_f32_kernel<G><<<grid, 256, 0, st>>>((const float*)a, lda, (const float*)w1, (const float*)w2, (float*)out, order, tile_expert, tile_start, tile_count, pair_weight, top, N, K, act)
    if (mode == 1) MOE_F32(1);
    else if (mode == 2) MOE_F32(2);
    else MOE_F32(0);
#undef MOE_F32
  }
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// stream[t][n] += sum over j < top of y[t * top + j][n], in ascending j. With ids: a choice whose id is `real` or more is
// an identity expert, and its term is weights[t * top + j] * x[t][n] (y holds nothing for it).
template <typename TX>
__global__ void moe_combine_kernel(float* __restrict__ stream, const float* __restrict__ y, int top, int N,
                                   const int* __restrict__ ids, const float* __restrict__ weights, const TX* __restrict__ x,
                                   int ldx, int real) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  const size_t t = blockIdx.y;
  float acc = 0.f;
  for (int j = 0; j < top; ++j) {
    if (ids != nullptr && ids[t * top + j] >= real) acc += weights[t * top + j] * to_f32(x[t * ldx + n]);
    else acc += y[(t * top + j) * N + n];
  }
  stream[t * N + n] += acc;
}

extern "C" int ms_moe_combine(float* stream, const float* y, int T, int top, int N, const int* ids, const float* weights,
                              const void* x, int x_is_bf16, int ldx, int real, hipStream_t st) {
  if (T <= 0 || N <= 0) return MS_OK;
  if (stream == nullptr || y == nullptr || top < 1 || T > 65535 || (ids != nullptr && (weights == nullptr || x == nullptr || ldx < N)))
    return MS_BAD_ARG;
  const dim3 grid((N + 255) / 256, T);
  if (x_is_bf16) moe_combine_kernel<bf16><<<grid, 256, 0, st>>>(stream, y, top, N, ids, weights, (const bf16*)x, ldx, real);
  else moe_combine_kernel<float><<<grid, 256, 0, st>>>(stream, y, top, N, ids, weights, (const float*)x, ldx, real);
  return launch_status();
}
