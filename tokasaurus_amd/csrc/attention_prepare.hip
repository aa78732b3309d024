// Between the q|k|v product and the attention, for mixers that norm queries and keys over
// the whole projection and rotate neighbouring elements: one kernel a step that
//   * divides a token's whole query row (all heads at once) by its root mean square and
//     multiplies by a weight of that size, and the same for its whole key row,
//   * rotates the leading `rot` elements of every head, element 2i with element 2i + 1, by the
//     angle position * freq[i] (32-bit product, 32-bit sine and cosine computed here: no table,
//     so positions have no upper end),
//   * writes the queries back in place, the keys and the values into the token's page.
// The arithmetic is 32-bit from the product's rounded output to the one rounding at the store.
//   row: [nq*dk | nkv*dk | nkv*dv]  (only the first part when !write_cache)
//   K pages: [page][kv head][dk / 8][P][8]    V pages: [page][kv head][P / 4][dv][4]
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void qk_prepare_kernel(
    T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
    const int* __restrict__ token_req, const int* __restrict__ block_table, int table_stride,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ freq, T* __restrict__ kcache, T* __restrict__ vcache, int nq, int nkv,
    int dk, int dv, int rot, int P, int write_cache) {
  extern __shared__ float cs[];  // [rot / 2] cosines, [rot / 2] sines
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot / 2;
  T* row = qkv + (size_t)t * row_stride;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float angle = __fmul_rn((float)pos, freq[i]);
    float s, c;
    sincosf(angle, &s, &c);
    cs[i] = c;
    cs[half + i] = s;
  }
  const int nqe = nq * dk, nke = nkv * dk;
  float rq = 1.f, rk = 1.f;
  if (q_weight) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nqe; i += blockDim.x) {
      const float v = to_f32<T>(row[i]);
      ss = fmaf(v, v, ss);
    }
    rq = 1.0f / sqrtf(block_sum(ss, red) / (float)nqe + eps);
  }
  if (write_cache && k_weight) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nke; i += blockDim.x) {
      const float v = to_f32<T>(row[nqe + i]);
      ss = fmaf(v, v, ss);
    }
    rk = 1.0f / sqrtf(block_sum(ss, red) / (float)nke + eps);
  }
  __syncthreads();  // the table of this token's angles is written

  // queries, in place, a pair of neighbours a thread (a head of odd size ends in a single element)
  const int hp = (dk + 1) / 2;
  for (int i = threadIdx.x; i < nq * hp; i += blockDim.x) {
    const int e = 2 * (i % hp), x = (i / hp) * dk + e;
    const bool two = e + 1 < dk;
    float u = to_f32<T>(row[x]) * rq, v = two ? to_f32<T>(row[x + 1]) * rq : 0.f;
    if (q_weight) {
      u *= q_weight[x];
      if (two) v *= q_weight[x + 1];
    }
    if (e < rot) rotate_pair(u, v, cs[e / 2], cs[half + e / 2], u, v);
    row[x] = from_f32<T>(u);
    if (two) row[x + 1] = from_f32<T>(v);
  }
  if (!write_cache) return;

  const int page = block_table[(size_t)token_req[t] * table_stride + pos / P];
  const int p = pos % P;
  const T* krow = row + nqe;
  const T* vrow = krow + nke;
  for (int i = threadIdx.x; i < nkv * hp; i += blockDim.x) {
    const int h = i / hp, e = 2 * (i % hp), x = h * dk + e;
    const bool two = e + 1 < dk;
    float u = to_f32<T>(krow[x]) * rk, v = two ? to_f32<T>(krow[x + 1]) * rk : 0.f;
    if (k_weight) {
      u *= k_weight[x];
      if (two) v *= k_weight[x + 1];
    }
    if (e < rot) rotate_pair(u, v, cs[e / 2], cs[half + e / 2], u, v);
    T* dst = kcache + ((size_t)page * nkv + h) * key_page_elems(P, dk);
    dst[key_offset(P, p, e)] = from_f32<T>(u);
    if (two) dst[key_offset(P, p, e + 1)] = from_f32<T>(v);
  }
  for (int i = threadIdx.x; i < nkv * dv; i += blockDim.x) {
    const int h = i / dv, e = i % dv;
    vcache[((size_t)page * nkv + h) * P * dv + value_offset(dv, p, e)] = vrow[i];
  }
}

TK_API int tk_qk_prepare(int dt, void* qkv, int row_stride, const int* positions, const int* token_req,
                         const int* block_table, int table_stride, const float* q_weight,
                         const float* k_weight, float eps, const float* freq, void* kcache, void* vcache,
                         int n_tokens, int nq, int nkv, int dk, int dv, int rot, int P, int write_cache,
                         hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && nq > 0 && nkv >= 0 && dk > 0 && dv > 0 && P > 0,
             "qk_prepare: bad sizes tokens=%d nq=%d nkv=%d dk=%d dv=%d P=%d", n_tokens, nq, nkv, dk, dv, P);
  TK_REQUIRE(rot >= 0 && rot <= dk && rot % 2 == 0, "qk_prepare: %d rotated elements of a head of %d", rot, dk);
  TK_REQUIRE(rot == 0 || freq, "qk_prepare: a rotation needs its frequencies");
  TK_REQUIRE(row_stride >= (write_cache ? nq * dk + nkv * (dk + dv) : nq * dk),
             "qk_prepare: row stride %d is shorter than the heads it holds", row_stride);
  TK_REQUIRE(!write_cache || (kcache && vcache && block_table && nkv > 0), "qk_prepare: cache pointers missing");
  if (n_tokens == 0) return 0;
  const size_t smem = sizeof(float) * (size_t)(rot > 0 ? rot : 2);
  if (dt == TK_F32)
    hipLaunchKernelGGL(qk_prepare_kernel<float>, dim3(n_tokens), dim3(256), smem, stream, (float*)qkv,
                       row_stride, positions, token_req, block_table, table_stride, q_weight, k_weight, eps,
                       freq, (float*)kcache, (float*)vcache, nq, nkv, dk, dv, rot, P, write_cache);
  else
    hipLaunchKernelGGL(qk_prepare_kernel<bf16_t>, dim3(n_tokens), dim3(256), smem, stream, (bf16_t*)qkv,
                       row_stride, positions, token_req, block_table, table_stride, q_weight, k_weight, eps,
                       freq, (bf16_t*)kcache, (bf16_t*)vcache, nq, nkv, dk, dv, rot, P, write_cache);
  TK_CHECK_LAUNCH("qk_prepare");
  return 0;
}
