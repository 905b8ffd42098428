// The recurrence with a decay per key channel and token and a bonus for the current token,
//     o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,     S_t = diag(w_t) S_(t-1) + k_t v_t^T          (S: [D, D] per head)
// for rows that bring many tokens, in chunks of WKV_CHUNK tokens and three passes, so that every chunk of every row and
// head has a block of its own. With l_t = log w_t (<= 0, per channel), A_t = l_0 + .. + l_t inside a chunk and
// B_t = A_(t-1) (B_0 = 0):
//   1. per chunk: its own contribution to the state at its end, U = sum_j diag(exp(A_last - A_j)) k_j v_j^T, and what
//      the chunk leaves of a state that enters it, G = exp(A_last);
//   2. per (row, head), chunk after chunk: the state *before* each chunk takes U's place in the buffer,
//      S' = diag(G) S + U; the state after the last chunk goes to the slot;
//   3. per chunk, with the state S0 before it:
//      o_t = S0^T (r_t * exp(B_t)) + sum_(j < t) P_tj v_j + (r_t . (u * k_t)) v_t,   P_tj = sum_d r_t[d] k_j[d] exp(B_t[d] - A_j[d]).
// Every exponent is a sum of log decays and so at most zero: nothing is ever divided by a decay. All float32; sums are
// reassociated against the token-by-token kernel (which multiplies by exp(l_t) token after token), nothing else differs;
// the exponentials are the hardware's exp2 of a float32 product (an error of a unit or two in the last place).
// The running sums are double precision: the kernels need their differences, and the difference of two sums that both hold
// one token's log of -100 (a channel that forgets everything there) must still be sharp for the tokens behind it; a float32
// sum of that size would leave those differences with an error of 1e-5. Logs arrive clamped at -200 a token (the decay is
// zero in float32 from -104 on), so a chunk's sums stay below 12,800. Head sizes up to WKV_CHUNK_MAX_DIM; larger ones take
// the token-by-token kernel.
#include "common.h"

#define WKV_CHUNK 64
#define WKV_CHUNK_MAX_DIM 64
#define WKV_CS (WKV_CHUNK + 4)  // floats between the rows of a transposed tile [channel][token]: rows stay 16-byte aligned, and
                                // the channels of one token, which one instruction stores, do not all fall into one bank

struct WkvChunkArgs {
  const float* x;  // [tokens, ld]: r, k and v of head h from columns r_off / k_off / v_off + h D on
  int ld, r_off, k_off, v_off, H, D;
  const float* lw;  // log decays [tokens, ld_w], head h's channels from column h D on
  int ld_w;
  const float* u;  // [H, D]
  float* S;        // [slots, H, D, D]
  const int* row_start;
  const int* starts;
  const int* state_slots;
  float* out;  // [tokens, H D]
  float* U;    // [chunks, H, D D]
  float* G;    // [chunks, H, D]
  int rows;
};

// The chunk `c` of the step: its row, first token and token count; *base = index of the row's first chunk.
__device__ __forceinline__ void wkv_find_chunk(const int* __restrict__ row_start, int rows, int c, int* row, int* first, int* count,
                                               int* base) {
  int b = 0, at = 0;
  for (; b < rows - 1; ++b) {
    const int nc = (row_start[b + 1] - row_start[b] + WKV_CHUNK - 1) / WKV_CHUNK;
    if (c < at + nc) break;
    at += nc;
  }
  *row = b;
  *base = at;
  *first = row_start[b] + (c - at) * WKV_CHUNK;
  const int left = row_start[b + 1] - *first;
  *count = left < WKV_CHUNK ? left : WKV_CHUNK;
}

// dst[d][t] = x[first + t][col + d] for t < count, d < D; zero elsewhere ([DP][WKV_CS]).
template <typename TD>
__device__ __forceinline__ void wkv_load_transposed(TD* dst, const float* __restrict__ x, int ld, int col, int first, int count, int D,
                                                    int DP) {
  for (int i = threadIdx.x; i < DP * WKV_CHUNK; i += blockDim.x) {
    const int t = i / DP, d = i % DP;  // consecutive threads read consecutive columns of one token
    dst[d * WKV_CS + t] = (TD)((t < count && d < D) ? x[(size_t)(first + t) * ld + col + d] : 0.f);
  }
}

// In place over L [DP][WKV_CS] of log decays: the running sums A_t (inclusive). A thread per channel, in token order.
__device__ __forceinline__ void wkv_running_sums(double* L, int DP) {
  if (threadIdx.x < DP) {
    double* row = L + threadIdx.x * WKV_CS;
    double run = 0.0;
    for (int t = 0; t < WKV_CHUNK; ++t) {
      run += row[t];
      row[t] = run;
    }
  }
}

__global__ __launch_bounds__(256) void wkv_chunk_summary_kernel(WkvChunkArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int D = a.D, h = blockIdx.y, tid = threadIdx.x;
  const int DP = (D + 3) & ~3;
  float* Kw = sm;                   // [WKV_CHUNK][DP]: keys times what is left of them at the chunk's end
  float* V = Kw + WKV_CHUNK * DP;   // [WKV_CHUNK][DP]
  double* A = reinterpret_cast<double*>(V + WKV_CHUNK * DP);  // [DP][WKV_CS] (8-byte aligned: both tiles are multiples of 4 floats)
  int row, first, count, base;
  wkv_find_chunk(a.row_start, a.rows, blockIdx.x, &row, &first, &count, &base);
  wkv_load_transposed(A, a.lw, a.ld_w, h * D, first, count, D, DP);
  for (int i = tid; i < WKV_CHUNK * DP; i += 256) {
    const int t = i / DP, d = i % DP;
    const bool ok = t < count && d < D;
    const float* xr = a.x + (size_t)(first + t) * a.ld;
    Kw[i] = ok ? xr[a.k_off + h * D + d] : 0.f;
    V[i] = ok ? xr[a.v_off + h * D + d] : 0.f;
  }
  __syncthreads();
  wkv_running_sums(A, DP);
  __syncthreads();
  for (int i = tid; i < WKV_CHUNK * DP; i += 256) {
    const int t = i / DP, d = i % DP;
    Kw[i] *= __expf((float)(A[d * WKV_CS + WKV_CHUNK - 1] - A[d * WKV_CS + t]));  // tokens past the count hold zero keys and zero logs
  }
  const size_t at = (size_t)blockIdx.x * a.H + h;
  if (tid < D) a.G[at * D + tid] = __expf((float)A[tid * WKV_CS + WKV_CHUNK - 1]);
  __syncthreads();
  // U[d][e]: 4 x 4 outputs a thread
  const int tiles = DP / 4;
  float* Ug = a.U + at * (size_t)D * D;
  for (int tile = tid; tile < tiles * tiles; tile += 256) {
    const int d0 = (tile / tiles) * 4, e0 = (tile % tiles) * 4;
    float acc[4][4] = {};
    for (int t = 0; t < WKV_CHUNK; ++t) {
      const float4 k4 = *reinterpret_cast<const float4*>(Kw + t * DP + d0);
      const float4 v4 = *reinterpret_cast<const float4*>(V + t * DP + e0);
      const float kk[4] = {k4.x, k4.y, k4.z, k4.w}, vv[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(kk[i], vv[j], acc[i][j]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (d0 + i < D && e0 + j < D) Ug[(size_t)(d0 + i) * D + e0 + j] = acc[i][j];
  }
}

__global__ __launch_bounds__(256) void wkv_chunk_scan_kernel(WkvChunkArgs a, int slices) {
  const int b = blockIdx.x, h = blockIdx.y, z = blockIdx.z, tid = threadIdx.x;
  const int D = a.D, DE = D * D;
  const int t0 = a.row_start[b], t1 = a.row_start[b + 1];
  const int nc = (t1 - t0 + WKV_CHUNK - 1) / WKV_CHUNK;
  int base = 0;
  for (int r = 0; r < b; ++r) base += (a.row_start[r + 1] - a.row_start[r] + WKV_CHUNK - 1) / WKV_CHUNK;
  const bool fresh = a.starts[b] == 0;
  float* Sg = a.S + ((size_t)a.state_slots[b] * a.H + h) * (size_t)DE;
  constexpr int PER = 8;
  float S[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = (z + slices * i) * 256 + tid;
    S[i] = (!fresh && idx < DE) ? Sg[idx] : 0.f;
  }
  for (int k = 0; k < nc; ++k) {
    const size_t at = (size_t)(base + k) * a.H + h;
    float* Uc = a.U + at * DE;
    const float* Gc = a.G + at * D;
    float t[PER], g[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = (z + slices * i) * 256 + tid;
      t[i] = idx < DE ? Uc[idx] : 0.f;
      g[i] = idx < DE ? Gc[idx / D] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = (z + slices * i) * 256 + tid;
      if (idx < DE) Uc[idx] = S[i];
      S[i] = fmaf(g[i], S[i], t[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = (z + slices * i) * 256 + tid;
    if (idx < DE) Sg[idx] = S[i];
  }
}

// Five waves a block: four for the tiles below the diagonal and everything else, the fifth for the sixteen tiles on it.
#define WKV_OUT_THREADS 320
__global__ __launch_bounds__(WKV_OUT_THREADS) void wkv_chunk_output_kernel(WkvChunkArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  constexpr int C = WKV_CHUNK, CP = WKV_CHUNK + 4, CS = WKV_CS;
  const int D = a.D, h = blockIdx.y, tid = threadIdx.x;
  const int DP = (D + 3) & ~3;
  double* A = reinterpret_cast<double*>(sm);  // [DP][CS]: running sums, inclusive
  double* Bx = A + DP * CS;                   // [DP][CS]: running sums, exclusive
  float* R = reinterpret_cast<float*>(Bx + DP * CS);  // [DP][CS]: r transposed; later r * exp(B)
  float* K = R + DP * CS;     // [DP][CS]
  float* V = K + DP * CS;     // [C][DP]
  float* P = V + C * DP;      // [C][CP]
  float* us = P + C * CP;     // [DP]
  int row, first, count, base;
  wkv_find_chunk(a.row_start, a.rows, blockIdx.x, &row, &first, &count, &base);
  wkv_load_transposed(R, a.x, a.ld, a.r_off + h * D, first, count, D, DP);
  wkv_load_transposed(K, a.x, a.ld, a.k_off + h * D, first, count, D, DP);
  wkv_load_transposed(Bx, a.lw, a.ld_w, h * D, first, count, D, DP);
  for (int i = tid; i < C * DP; i += WKV_OUT_THREADS) {
    const int t = i / DP, d = i % DP;
    V[i] = (t < count && d < D) ? a.x[(size_t)(first + t) * a.ld + a.v_off + h * D + d] : 0.f;
  }
  if (tid < DP) us[tid] = tid < D ? a.u[h * D + tid] : 0.f;
  __syncthreads();
  if (tid < DP) {
    double run = 0.0;
    for (int t = 0; t < C; ++t) {
      const double l = Bx[tid * CS + t];
      Bx[tid * CS + t] = run;
      run += l;
      A[tid * CS + t] = run;
    }
  }
  __syncthreads();
  // P: 4 x 4 entries a thread. A tile below the diagonal (all its keys before all its tokens) splits every exponential at
  // the tile's last key m: exp(B_t - A_j) = exp(B_t - A_m) exp(A_m - A_j), both exponents sums of log decays and so at most
  // zero: eight exponentials for sixteen terms. A tile on the diagonal has six terms with j < t and the bonus where j == t;
  // those sixteen tiles are the fifth wave's, so that no wave walks both forms. Tiles above the diagonal hold nothing.
  {
    float acc[4][4] = {};
    const bool low = tid < 256;
    const int ti = low ? tid / 16 : tid - 256, ji = low ? tid % 16 : tid - 256;  // 16 x 16 tiles of 4 x 4
    const int t0 = ti * 4, j0 = ji * 4;
    const bool mine = low ? ji != ti : ti < 16;
    if (mine && ji <= ti && t0 < count) {
      for (int d = 0; d < D; ++d) {
        const float4 r4 = *reinterpret_cast<const float4*>(R + d * CS + t0);
        const float4 k4 = *reinterpret_cast<const float4*>(K + d * CS + j0);
        const double2 b01 = *reinterpret_cast<const double2*>(Bx + d * CS + t0), b23 = *reinterpret_cast<const double2*>(Bx + d * CS + t0 + 2);
        const double2 a01 = *reinterpret_cast<const double2*>(A + d * CS + j0), a23 = *reinterpret_cast<const double2*>(A + d * CS + j0 + 2);
        const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w};
        const double bb[4] = {b01.x, b01.y, b23.x, b23.y}, aa[4] = {a01.x, a01.y, a23.x, a23.y};
        if (low) {
          float rf[4], kf[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) rf[i] = rr[i] * __expf((float)(bb[i] - aa[3]));
#pragma unroll
          for (int j = 0; j < 3; ++j) kf[j] = kk[j] * __expf((float)(aa[3] - aa[j]));
          kf[3] = kk[3];
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(rf[i], kf[j], acc[i][j]);
        } else {
          const float ud = us[d];
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j <= i; ++j) {
              // j < t: what is left of key j's channel when token t reads it; j == t: the bonus
              const float wgt = j < i ? __expf((float)(bb[i] - aa[j])) : ud;
              acc[i][j] = fmaf(rr[i] * kk[j], wgt, acc[i][j]);
            }
        }
      }
    }
    if (mine)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<float4*>(P + (t0 + i) * CP + j0) = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
  }
  __syncthreads();
  for (int i = tid; i < DP * C; i += WKV_OUT_THREADS) {  // what of the state before the chunk token t still reads
    const int at = (i / C) * CS + i % C;
    R[at] *= __expf((float)Bx[at]);
  }
  __syncthreads();
  // The state before the chunk takes the keys' place in LDS: [D][DP], zero beyond D.
  {
    const float* S0g = a.U + ((size_t)blockIdx.x * a.H + h) * (size_t)D * D;
    for (int i = tid; i < D * DP; i += WKV_OUT_THREADS) {
      const int d = i / DP, e = i % DP;
      K[i] = e < D ? S0g[(size_t)d * D + e] : 0.f;
    }
  }
  __syncthreads();
  // o[t][e]: 4 x 4 outputs a thread
  const float* S0 = K;
  const int etiles = DP / 4;
  for (int tile = tid; tile < (C / 4) * etiles; tile += WKV_OUT_THREADS) {
    const int t0 = (tile / etiles) * 4, e0 = (tile % etiles) * 4;
    if (t0 >= count) continue;
    float o[4][4] = {};
    for (int d = 0; d < D; ++d) {
      const float4 r4 = *reinterpret_cast<const float4*>(R + d * CS + t0);
      const float rr[4] = {r4.x, r4.y, r4.z, r4.w};
      const float4 s4 = *reinterpret_cast<const float4*>(S0 + d * DP + e0);
      const float sv[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) o[i][j] = fmaf(rr[i], sv[j], o[i][j]);
    }
    const int jend = t0 + 4 < count ? t0 + 4 : count;
    for (int jj = 0; jj < jend; ++jj) {
      const float4 v4 = *reinterpret_cast<const float4*>(V + jj * DP + e0);
      const float vv[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = P[(t0 + i) * CP + jj];
#pragma unroll
        for (int j = 0; j < 4; ++j) o[i][j] = fmaf(p, vv[j], o[i][j]);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (t0 + i < count && e0 + j < D) a.out[(size_t)(first + t0 + i) * (a.H * D) + h * D + e0 + j] = o[i][j];
  }
}

extern "C" int ms_wkv_chunk_tokens() { return WKV_CHUNK; }
extern "C" int ms_wkv_chunk_max_dim() { return WKV_CHUNK_MAX_DIM; }

// x, lw, u, S, the rows and out as for the token-by-token kernel (lw: the decays' logarithms). `chunks` = sum over the rows
// of ceil(tokens / WKV_CHUNK) (the host knows the rows' lengths); U [chunks, H, D D] and G [chunks, H, D] are scratch.
extern "C" int ms_wkv_chunked(const float* x, int ld, int r_off, int k_off, int v_off, int H, int D, const float* lw, int ld_w,
                              const float* u, float* S, const int* row_start, const int* starts, const int* state_slots, float* out,
                              int rows, int chunks, float* U, float* G, hipStream_t st) {
  if (rows <= 0 || chunks <= 0) return MS_OK;
  if (H <= 0 || D <= 0 || x == nullptr || lw == nullptr || u == nullptr || S == nullptr || out == nullptr || row_start == nullptr ||
      starts == nullptr || state_slots == nullptr || U == nullptr || G == nullptr || r_off < 0 || k_off < 0 || v_off < 0 ||
      r_off + H * D > ld || k_off + H * D > ld || v_off + H * D > ld || ld_w < H * D)
    return MS_BAD_ARG;
  if (D > WKV_CHUNK_MAX_DIM || H > 65535 || rows > 65535) return MS_UNSUPPORTED;
  WkvChunkArgs a{x, ld, r_off, k_off, v_off, H, D, lw, ld_w, u, S, row_start, starts, state_slots, out, U, G, rows};
  const int DP = (D + 3) & ~3;
  const size_t lds1 = sizeof(float) * (size_t)(2 * WKV_CHUNK * DP + 2 * DP * WKV_CS);  // a double takes two floats' room
  const size_t lds3 = sizeof(float) * (size_t)(6 * DP * WKV_CS + WKV_CHUNK * DP + WKV_CHUNK * (WKV_CHUNK + 4) + DP);
  if (hipFuncSetAttribute((const void*)wkv_chunk_summary_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds1) != hipSuccess ||
      hipFuncSetAttribute((const void*)wkv_chunk_output_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds3) != hipSuccess)
    return MS_LAUNCH_FAILED;
  wkv_chunk_summary_kernel<<<dim3(chunks, H), 256, lds1, st>>>(a);
  const int slices = (D * D + 256 * 8 - 1) / (256 * 8);
  wkv_chunk_scan_kernel<<<dim3(rows, H, slices), 256, 0, st>>>(a, slices);
  wkv_chunk_output_kernel<<<dim3(chunks, H), WKV_OUT_THREADS, lds3, st>>>(a);
  return launch_status();
}
