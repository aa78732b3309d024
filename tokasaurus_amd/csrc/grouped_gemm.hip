// Matrix products in which every tile of rows has a weight matrix of its own, on
// v_mfma_f32_16x16x32_bf16: the experts of a mixture (rows sorted by expert) and a matrix a head.
//
//   tk_expert_sort        pairs (token, chosen expert) sorted by expert into slots, every expert's
//                         run of slots filled up to whole tiles of GG_TM slots
//   tk_grouped_gemm_bf16  C[c_row(slot), g * c_cols + n] = sum_k W[g][n][k] * A[a_row(slot), g * a_cols + k]
//                         for the slots of every tile, g the tile's group; optionally the gated form
//                         silu(gate) * up of two halves of W[g]
//   tk_expert_sum         per token the weighted sum of its pairs' rows, identity experts, shared expert
//
// A wavefront owns GG_TM = 64 slots x 64 outputs (32 in the gated form, for each of gate and up): weight rows
// are the first operand of the matrix core, read straight from memory 16 bytes a lane, the slots' rows the
// second; a lane ends up with 4 neighbouring outputs of one slot.  The next step's operands are asked for
// before the current step's products.  Sums are 32-bit and run over k in ascending order for every output:
// a row's result does not depend on which other rows share its tile.
#include <math.h>

#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define GG_TM 64
#define GG_WAVES 4

__device__ __forceinline__ bf16x8_t gg_zero8() {
  bf16x8_t z;
#pragma unroll
  for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.f;
  return z;
}

struct GroupedArgs {
  const bf16_t* A;
  int lda;
  const int* a_row;       // [slots] the row of A a slot reads, < 0: an empty slot; null: the slot's own number
  const int* c_row;       // [slots] the row of C a slot writes, < 0: none; null: the slot's own number
  const int* tile_group;  // [tiles] the group of every tile of GG_TM slots, < 0: an unused tile; null: blockIdx.z
  int a_cols, c_cols;     // columns of A and C that a group is offset by
  const bf16_t* W;        // [groups][N (2 N in the gated form: gate rows, then up rows)][K]
  size_t w_stride;        // elements from one group's matrix to the next
  void* C;
  int ldc;
  int N, K, slots;
};

// NT: blocks of 16 outputs a wavefront; GLU: the gated form; F32: 32-bit output
template <int NT, bool GLU, bool F32>
__global__ __launch_bounds__(GG_WAVES * TK_WAVE) void grouped_gemm_kernel(GroupedArgs a) {
  constexpr int MB = GG_TM / 16;
  constexpr int WT = GLU ? 2 * NT : NT;  // weight blocks a wavefront reads a step
  const int lane = threadIdx.x & (TK_WAVE - 1), wave = threadIdx.x / TK_WAVE;
  const int tile = blockIdx.x;
  const int g = a.tile_group ? a.tile_group[tile] : (int)blockIdx.z;
  if (g < 0) return;
  const int n0 = (blockIdx.y * GG_WAVES + wave) * NT * 16;
  if (n0 >= a.N) return;
  const int r = lane & 15, q = lane >> 4;
  const bf16_t* Wg = a.W + (size_t)g * a.w_stride;
  const bf16_t* wp[WT];
#pragma unroll
  for (int t = 0; t < WT; ++t) {
    const int blk = GLU ? t % NT : t;
    const int row = min(n0 + blk * 16 + r, a.N - 1) + ((GLU && t >= NT) ? a.N : 0);
    wp[t] = Wg + (size_t)row * a.K + q * 8;
  }
  const bf16_t* ap[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int slot = tile * GG_TM + mb * 16 + r;
    int row = slot < a.slots ? (a.a_row ? a.a_row[slot] : slot) : -1;
    ap[mb] = a.A + (size_t)max(row, 0) * a.lda + (size_t)g * a.a_cols + q * 8;
  }
  f32x4_t acc[WT][MB];
#pragma unroll
  for (int t = 0; t < WT; ++t)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[t][mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int steps = (a.K + 31) / 32;
  bf16x8_t w[WT], av[MB];
  auto load = [&](int ks, bf16x8_t (&wv)[WT], bf16x8_t (&xv)[MB]) {
    // a step may reach past K (a multiple of 8): read a valid chunk and zero the weight
    const bool k_ok = ks * 32 + q * 8 < a.K;
    const long off = k_ok ? (long)ks * 32 : -(long)(q * 8);
#pragma unroll
    for (int t = 0; t < WT; ++t) {
      wv[t] = *(const bf16x8_t*)(wp[t] + off);
      if (!k_ok) wv[t] = gg_zero8();
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) xv[mb] = *(const bf16x8_t*)(ap[mb] + off);
  };
  load(0, w, av);
  for (int ks = 0; ks < steps; ++ks) {
    bf16x8_t wn[WT], an[MB];
    if (ks + 1 < steps) load(ks + 1, wn, an);
#pragma unroll
    for (int t = 0; t < WT; ++t)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        acc[t][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[t], av[mb], acc[t][mb], 0, 0, 0);
    if (ks + 1 < steps) {
#pragma unroll
      for (int t = 0; t < WT; ++t) w[t] = wn[t];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) av[mb] = an[mb];
    }
  }
  // lane: slot mb * 16 + r, outputs n0 + t * 16 + 4 q + j
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int slot = tile * GG_TM + mb * 16 + r;
    if (slot >= a.slots) continue;
    if (a.a_row && a.a_row[slot] < 0) continue;
    const int crow = a.c_row ? a.c_row[slot] : slot;
    if (crow < 0) continue;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = n0 + t * 16 + 4 * q;
      float y[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) y[j] = GLU ? silu_mul_bf16(acc[t][mb][j], acc[t + (GLU ? NT : 0)][mb][j]) : acc[t][mb][j];
      const size_t at = (size_t)crow * a.ldc + (size_t)g * a.c_cols + n;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (n + j < a.N) {
          if (F32) ((float*)a.C)[at + j] = y[j];
          else ((bf16_t*)a.C)[at + j] = __float2bfloat16(y[j]);
        }
      }
    }
  }
}

TK_API int tk_grouped_gemm_bf16(const void* A, int lda, const int* a_row, const int* c_row, const int* tile_group, int tiles,
                                int groups_z, int a_cols, int c_cols, const void* W, size_t w_stride, void* C, int ldc,
                                int N, int K, int slots, int glu, int out_f32, hipStream_t stream) {
  TK_REQUIRE(A && W && C && N > 0 && K > 0 && slots >= 0 && tiles >= 0, "grouped_gemm: bad arguments");
  TK_REQUIRE(K % 8 == 0 && lda % 8 == 0 && a_cols % 8 == 0 && w_stride % 8 == 0 && (((uintptr_t)A | (uintptr_t)W) & 15) == 0,
             "grouped_gemm: rows of A and W must start at multiples of 16 bytes (K=%d lda=%d)", K, lda);
  TK_REQUIRE((tile_group != nullptr) != (groups_z > 0), "grouped_gemm: groups come by tile or by the grid, not both");
  TK_REQUIRE(!(glu && out_f32), "grouped_gemm: the gated form writes the storage type");
  if (tiles == 0 || slots == 0) return 0;
  GroupedArgs a{(const bf16_t*)A, lda, a_row, c_row, tile_group, a_cols, c_cols, (const bf16_t*)W, w_stride, C, ldc, N, K, slots};
  const int nt = glu ? 2 : 4;
  const dim3 grid(tiles, (N + GG_WAVES * nt * 16 - 1) / (GG_WAVES * nt * 16), groups_z > 0 ? groups_z : 1);
  TK_REQUIRE(grid.y < 65536 && grid.z < 65536, "grouped_gemm: too many outputs or groups");
  if (glu)
    hipLaunchKernelGGL((grouped_gemm_kernel<2, true, false>), grid, dim3(GG_WAVES * TK_WAVE), 0, stream, a);
  else if (out_f32)
    hipLaunchKernelGGL((grouped_gemm_kernel<4, false, true>), grid, dim3(GG_WAVES * TK_WAVE), 0, stream, a);
  else
    hipLaunchKernelGGL((grouped_gemm_kernel<4, false, false>), grid, dim3(GG_WAVES * TK_WAVE), 0, stream, a);
  TK_CHECK_LAUNCH("grouped_gemm");
  return 0;
}

// --------------------------------------------------------------------------
// Pairs (token, place) -> slots sorted by expert.  One workgroup.  Expert e's pairs take the slots
// first[e] .. first[e] + count[e] - 1 with first[e] a multiple of GG_TM; the slots between a run's end and the
// next multiple are empty.  slot_pair[slot] = the pair (or -1), slot_token[slot] = its token (or -1),
// tile_group[tile] = the expert whose run the tile lies in (or -1).  Pairs of identity experts (ids >= experts)
// and empty places (ids < 0) get no slot.  Which of an expert's slots a pair gets depends on the order of
// arrival and changes no result: every row is computed on its own.
// --------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void expert_sort_kernel(const int* __restrict__ ids, int pairs, int top, int experts,
                                                           int max_tiles, int* __restrict__ slot_pair,
                                                           int* __restrict__ slot_token, int* __restrict__ tile_group) {
  extern __shared__ int sh[];  // [experts] counts, [experts] first slots, [experts] cursors
  int* count = sh;
  int* first = sh + experts;
  int* cursor = sh + 2 * experts;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = cursor[e] = 0;
  for (int s = threadIdx.x; s < max_tiles * GG_TM; s += blockDim.x) slot_pair[s] = slot_token[s] = -1;
  for (int t = threadIdx.x; t < max_tiles; t += blockDim.x) tile_group[t] = -1;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = at;
      at += (count[e] + GG_TM - 1) / GG_TM * GG_TM;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < experts; e += blockDim.x)
    for (int t = first[e] / GG_TM; t < (first[e] + count[e] + GG_TM - 1) / GG_TM; ++t) tile_group[t] = e;
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < experts) {
      const int s = first[e] + atomicAdd(&cursor[e], 1);
      slot_pair[s] = p;
      slot_token[s] = p / top;
    }
  }
}

TK_API int tk_expert_sort(const int* ids, int pairs, int top, int experts, int max_tiles, int* slot_pair, int* slot_token,
                          int* tile_group, hipStream_t stream) {
  TK_REQUIRE(ids && slot_pair && slot_token && tile_group && pairs >= 0 && top > 0 && experts > 0, "expert_sort: bad arguments");
  TK_REQUIRE(max_tiles >= (pairs + GG_TM - 1) / GG_TM + experts, "expert_sort: %d tiles cannot hold %d pairs of %d experts", max_tiles,
             pairs, experts);
  TK_REQUIRE(3 * experts * sizeof(int) <= 48 * 1024, "expert_sort: too many experts");
  hipLaunchKernelGGL(expert_sort_kernel, dim3(1), dim3(1024), 3 * experts * sizeof(int), stream, ids, pairs, top, experts,
                     max_tiles, slot_pair, slot_token, tile_group);
  TK_CHECK_LAUNCH("expert_sort");
  return 0;
}

// --------------------------------------------------------------------------
// out[t, c] = sum over the places k of token t, in order, of weights[t, k] * (y[t * top + k, c] for a routed expert,
// h[t, c] for an identity expert), plus shared_gate[t] * shared[t, c].  y: [pairs, width] in the storage type.
// --------------------------------------------------------------------------
__global__ __launch_bounds__(256) void expert_sum_kernel(const bf16_t* __restrict__ h, int h_stride, const bf16_t* __restrict__ y,
                                                         const int* __restrict__ ids, const float* __restrict__ weights,
                                                         const float* __restrict__ shared, const float* __restrict__ shared_gate,
                                                         float* __restrict__ out, int width, int experts, int top) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = ids[(size_t)t * top + k];
      if (e < 0) continue;
      const float v = e < experts ? __bfloat162float(y[((size_t)t * top + k) * width + c]) : __bfloat162float(h[(size_t)t * h_stride + c]);
      acc = fmaf(weights[(size_t)t * top + k], v, acc);
    }
    if (shared) acc = fmaf(shared_gate[t], shared[(size_t)t * width + c], acc);
    out[(size_t)t * width + c] = acc;
  }
}

TK_API int tk_expert_sum(const void* h, int h_stride, const void* y, const int* ids, const float* weights, const float* shared,
                         const float* shared_gate, float* out, int tokens, int width, int experts, int top, hipStream_t stream) {
  TK_REQUIRE(h && y && ids && weights && out && (!shared || shared_gate) && tokens >= 0 && width > 0 && top > 0 && h_stride >= width,
             "expert_sum: bad arguments");
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(expert_sum_kernel, dim3(tokens), dim3(256), 0, stream, (const bf16_t*)h, h_stride, (const bf16_t*)y, ids,
                     weights, shared, shared_gate, out, width, experts, top);
  TK_CHECK_LAUNCH("expert_sum");
  return 0;
}
