// Products in groups: Y_g = X_g * W_g^T for g = 0 .. G-1, one launch for all groups.
//
// A group is a head (every group has the same rows, its operands are column ranges of
// wider rows: the per-head projections of a latent attention) or an expert of a mixture
// (the groups' rows are slices of one sorted list of (token, choice) pairs whose bounds
// are on the device; rows of X are gathered and rows of Y scattered through index
// arrays).  W is [G, N, K] with row length ldw.  The epilogue can multiply by the sigmoid
// of a float32 gate (heads), or compute the clamped gated activation of two products
// (experts: W the gate's weight, W2 the up projection's), write float32 or bf16, or add
// into a float32 destination.  Accumulation is float32 throughout; a row's result depends
// on that row alone.
//
// Two kernels: tiles of 64 x 64 on the vector units for any element type and any sizes,
// and for bf16 operands whose addresses allow 16-byte loads the same tiles on the matrix
// cores (v_mfma_f32_16x16x32_bf16), operands read from memory in the instruction's own
// order.
#include "hal_common.h"
#include "hal_api.h"

struct GroupedArgs {
  const void* X;
  int ldx, x_group_cols, x_col0;
  const void* W;
  const void* W2;
  long long w_group_stride;
  int ldw;
  void* Y;
  int ldy, y_group_cols, y_col0, y_dtype, y_add;
  int M, N, K, G;
  const int* group_offsets;  // [G + 1] or null
  const int* tile_offsets;   // [G + 1] with group_offsets
  const int* row_src;        // or null
  int src_div;
  const int* row_dst;  // or null
  const float* gate;   // or null
  int ldg;
  float limit, alpha;
};

#define GG_TM 64
#define GG_TN 64
#define GG_TK 16

// which group and which rows a workgroup serves; false: nothing
__device__ __forceinline__ bool gg_locate(const GroupedArgs& a, int& g, int& row0, int& row_end) {
  if (a.group_offsets == nullptr) {
    g = blockIdx.z;
    row0 = blockIdx.y * GG_TM;
    row_end = a.M;
    return row0 < row_end;
  }
  const int tile = blockIdx.y;
  if (tile >= a.tile_offsets[a.G]) return false;
  int lo = 0, hi = a.G;  // the last group whose first tile is <= tile
  while (hi - lo > 1) {
    const int mid = (lo + hi) / 2;
    if (a.tile_offsets[mid] <= tile) lo = mid; else hi = mid;
  }
  g = lo;
  row0 = a.group_offsets[g] + (tile - a.tile_offsets[g]) * GG_TM;
  row_end = a.group_offsets[g + 1];
  return row0 < row_end;
}

__device__ __forceinline__ float gg_sigmoid(float z) { return 1.0f / (1.0f + __expf(-z)); }

__device__ __forceinline__ void gg_store(const GroupedArgs& a, int g, int i, int n, float v, float v2,
                                         bool gated) {
  if (gated) {
    const float gg = fminf(v, a.limit);
    const float uu = fminf(fmaxf(v2, -a.limit), a.limit);
    v = gg * gg_sigmoid(a.alpha * gg) * (uu + 1.0f);
  }
  const int dst = a.row_dst ? a.row_dst[i] : i;
  const size_t col = (size_t)g * a.y_group_cols + a.y_col0 + n;
  if (a.gate) v *= gg_sigmoid(a.gate[(size_t)dst * a.ldg + (size_t)g * a.y_group_cols + n]);
  const size_t at = (size_t)dst * a.ldy + col;
  if (a.y_dtype == HAL_F32) {
    float* y = (float*)a.Y;
    y[at] = a.y_add ? y[at] + v : v;
  } else {
    ((bf16_t*)a.Y)[at] = f32_to_bf16(v);
  }
}

template <typename T, bool GATED>
__global__ void __launch_bounds__(256) grouped_fma_kernel(GroupedArgs a) {
  int g, row0, row_end;
  if (!gg_locate(a, g, row0, row_end)) return;
  const int n0 = blockIdx.x * GG_TN;
  __shared__ float As[GG_TK][GG_TM + 4];
  __shared__ float Bs[GG_TK][GG_TN + 4];
  __shared__ float B2s[GATED ? GG_TK : 1][GG_TN + 4];
  __shared__ int src_rows[GG_TM];
  const int tid = threadIdx.x;
  if (tid < GG_TM) {
    const int i = row0 + tid;
    int s = -1;
    if (i < row_end) s = a.row_src ? a.row_src[i] / a.src_div : i;
    src_rows[tid] = s;
  }
  __syncthreads();
  const T* X = (const T*)a.X + (size_t)g * a.x_group_cols + a.x_col0;
  const T* W = (const T*)a.W + (size_t)g * a.w_group_stride;
  const T* W2 = GATED ? (const T*)a.W2 + (size_t)g * a.w_group_stride : nullptr;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4] = {}, acc2[4][4] = {};
  // a thread brings element (r, kk) of each tile, r = tid / 4 (+ 0), kk = (tid % 4) * 4 .. + 3
  const int lr = tid / 4, lk = (tid % 4) * 4;
  for (int k0 = 0; k0 < a.K; k0 += GG_TK) {
    const int s = src_rows[lr];
    const int n = n0 + lr;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      const bool kin = k < a.K;
      As[lk + j][lr] = (s >= 0 && kin) ? to_f32(X[(size_t)s * a.ldx + k]) : 0.f;
      Bs[lk + j][lr] = (n < a.N && kin) ? to_f32(W[(size_t)n * a.ldw + k]) : 0.f;
      if (GATED) B2s[lk + j][lr] = (n < a.N && kin) ? to_f32(W2[(size_t)n * a.ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GG_TK; ++kk) {
      float av[4], bv[4], b2v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = As[kk][tm + i];
        bv[i] = Bs[kk][tn + i];
        if (GATED) b2v[i] = B2s[kk][tn + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
          if (GATED) acc2[i][j] = fmaf(av[i], b2v[j], acc2[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + tm + i;
    if (r >= row_end) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tn + j;
      if (n < a.N) gg_store(a, g, r, n, acc[i][j], acc2[i][j], GATED);
    }
  }
}

typedef __attribute__((ext_vector_type(8))) __bf16 gg_bf16x8;
typedef __attribute__((ext_vector_type(4))) float gg_f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t gg_u32x4;

__device__ __forceinline__ gg_bf16x8 gg_frag(const bf16_t* p, bool valid) {
  gg_u32x4 raw = {0u, 0u, 0u, 0u};
  if (valid) raw = *(const gg_u32x4*)p;
  return __builtin_bit_cast(gg_bf16x8, raw);
}

// bf16 on the matrix cores.  Four waves; wave w takes rows 16w .. 16w + 15 of the tile and
// all of its 64 columns.  Lane l of an operand holds row l % 16 and the eight k from
// (l / 16) * 8 on; lane l of a result holds X row l % 16 and W rows 4 * (l / 16) .. + 3.
// K, ldx, ldw and the column offsets are multiples of 8 and the bases 16-byte aligned.
template <bool GATED>
__global__ void __launch_bounds__(256) grouped_mfma_kernel(GroupedArgs a) {
  int g, row0, row_end;
  if (!gg_locate(a, g, row0, row_end)) return;
  const int n0 = blockIdx.x * GG_TN;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int r = lane % 16, q = lane / 16;
  const bf16_t* X = (const bf16_t*)a.X + (size_t)g * a.x_group_cols + a.x_col0;
  const bf16_t* W = (const bf16_t*)a.W + (size_t)g * a.w_group_stride;
  const bf16_t* W2 = GATED ? (const bf16_t*)a.W2 + (size_t)g * a.w_group_stride : nullptr;
  const int i = row0 + wave * 16 + r;
  const bool xin = i < row_end;
  int s = 0;
  if (xin) s = a.row_src ? a.row_src[i] / a.src_div : i;
  const bf16_t* xrow = X + (size_t)s * a.ldx + q * 8;
  const bf16_t* wrow[4];
  const bf16_t* w2row[4];
  bool win[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int n = n0 + t * 16 + r;
    win[t] = n < a.N;
    wrow[t] = W + (size_t)(win[t] ? n : 0) * a.ldw + q * 8;
    w2row[t] = GATED ? W2 + (size_t)(win[t] ? n : 0) * a.ldw + q * 8 : nullptr;
  }
  gg_f32x4 acc[4], acc2[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    acc[t] = gg_f32x4{0.f, 0.f, 0.f, 0.f};
    acc2[t] = gg_f32x4{0.f, 0.f, 0.f, 0.f};
  }
  for (int k0 = 0; k0 < a.K; k0 += 64) {
    gg_bf16x8 xa[2], wa[2][4], w2a[2][4];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int k = k0 + u * 32;
      const bool kin = k + q * 8 < a.K;
      xa[u] = gg_frag(xrow + k, kin && xin);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        wa[u][t] = gg_frag(wrow[t] + k, kin && win[t]);
        if (GATED) w2a[u][t] = gg_frag(w2row[t] + k, kin && win[t]);
      }
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[u][t], xa[u], acc[t], 0, 0, 0);
        if (GATED) acc2[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w2a[u][t], xa[u], acc2[t], 0, 0, 0);
      }
  }
  if (!xin) return;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + t * 16 + q * 4 + j;
      if (n < a.N) gg_store(a, g, i, n, acc[t][j], acc2[t][j], GATED);
    }
}

extern "C" int hal_grouped_gemm(const void* X, int ldx, int x_group_cols, int x_col0, const void* W,
                                const void* W2, long long w_group_stride, int ldw, int dtype,
                                void* Y, int ldy, int y_group_cols, int y_col0, int y_dtype,
                                int y_add, int M, int N, int K, int G, const int* group_offsets,
                                const int* tile_offsets, const int* row_src, int src_div,
                                const int* row_dst, const float* gate, int ldg, float limit,
                                float alpha, int allow_mfma, hipStream_t stream) {
  HAL_REQUIRE(M >= 0 && N > 0 && K > 0 && G > 0, "hal_grouped_gemm: bad sizes M=%d N=%d K=%d G=%d", M, N,
              K, G);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_grouped_gemm: operand dtype %d", dtype);
  HAL_REQUIRE(y_dtype == HAL_F32 || y_dtype == HAL_BF16, "hal_grouped_gemm: result dtype %d", y_dtype);
  HAL_REQUIRE(!y_add || y_dtype == HAL_F32, "hal_grouped_gemm: only a float32 result is added into");
  HAL_REQUIRE((group_offsets == nullptr) == (tile_offsets == nullptr),
              "hal_grouped_gemm: group and tile offsets come together");
  HAL_REQUIRE(src_div > 0, "hal_grouped_gemm: src_div %d", src_div);
  HAL_REQUIRE(G <= 65535, "hal_grouped_gemm: %d groups", G);
  if (M == 0) return 0;
  GroupedArgs a;
  a.X = X; a.ldx = ldx; a.x_group_cols = x_group_cols; a.x_col0 = x_col0;
  a.W = W; a.W2 = W2; a.w_group_stride = w_group_stride; a.ldw = ldw;
  a.Y = Y; a.ldy = ldy; a.y_group_cols = y_group_cols; a.y_col0 = y_col0; a.y_dtype = y_dtype;
  a.y_add = y_add;
  a.M = M; a.N = N; a.K = K; a.G = G;
  a.group_offsets = group_offsets; a.tile_offsets = tile_offsets;
  a.row_src = row_src; a.src_div = src_div; a.row_dst = row_dst;
  a.gate = gate; a.ldg = ldg; a.limit = limit; a.alpha = alpha;
  const int row_tiles = (M + GG_TM - 1) / GG_TM;
  dim3 grid((N + GG_TN - 1) / GG_TN, group_offsets ? row_tiles + G : row_tiles, group_offsets ? 1 : G);
  HAL_REQUIRE(grid.y <= 65535, "hal_grouped_gemm: %u row tiles", grid.y);
  const bool aligned = K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && x_group_cols % 8 == 0 &&
                       x_col0 % 8 == 0 && w_group_stride % 8 == 0 && ((uintptr_t)X % 16 == 0) &&
                       ((uintptr_t)W % 16 == 0) && (W2 == nullptr || (uintptr_t)W2 % 16 == 0);
  if (dtype == HAL_BF16 && allow_mfma && aligned) {
    if (W2) hipLaunchKernelGGL(grouped_mfma_kernel<true>, grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(grouped_mfma_kernel<false>, grid, dim3(256), 0, stream, a);
  } else if (dtype == HAL_BF16) {
    if (W2) hipLaunchKernelGGL((grouped_fma_kernel<bf16_t, true>), grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((grouped_fma_kernel<bf16_t, false>), grid, dim3(256), 0, stream, a);
  } else {
    if (W2) hipLaunchKernelGGL((grouped_fma_kernel<float, true>), grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((grouped_fma_kernel<float, false>), grid, dim3(256), 0, stream, a);
  }
  HAL_LAUNCH_CHECK();
  return 0;
}
