// The gated delta rule with one decay per head and key channel, as a recurrence over the
// tokens of each request, and what stands around it: the short causal convolutions of q, k
// and v with their activation, the unit norms, the write strength and the decays (before), the
// per-head norm with its gate (after).  Everything that enters the recurrence is 32-bit.
//
// Per request a state row of 32-bit floats lives in the request's slot:
//   [ S: heads x dv x dk ][ tail: (taps - 1) x channels ]
// S is kept transposed (a value column's dk numbers lie together); the tail holds the last
// taps - 1 inputs of the convolutions, oldest first, channels = 2 * kv_heads * dk + heads * dv
// in the order q | k | v.  A slot's row is all zeros when a request takes it.
//
// Per token and head, with decay g (dk), write strength beta, unit k, scaled unit q, value v:
//   S <- diag(g) S;  u = beta * (v - S^T k);  S <- S + k u^T;  o = S^T q.
// The columns of S (one a value channel) do not meet: a column is owned by DR_LANES lanes that
// cut dk between them and add up through the wavefront, always in the same order, so a token's
// result does not depend on how its request's tokens were cut into steps or what shares the batch.
#include "common.h"

#define DR_LANES 8     // lanes that share a column of the state
#define DR_TOKENS 16   // tokens staged in LDS at a time
#define DR_MAX_TAPS 16

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f32(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// --------------------------------------------------------------------------
// Before the recurrence: one workgroup a token.
//   proj row (T): [q | k | v] (channels) ... and the write strength's `heads` numbers at col_b
//   a_pre (32-bit) [tokens, heads * dk]: the decay's projection before bias and softplus
//   rec row (32-bit): [q: G*dk | k: G*dk | v: H*dv | decay: H*dk | beta: H]
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_kernel(
    const T* __restrict__ proj, int ld, int col_b, const float* __restrict__ a_pre,
    const float* __restrict__ conv_w, int taps, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, const float* __restrict__ state, size_t state_stride,
    size_t tail_off, const int* __restrict__ q_start, const int* __restrict__ token_req,
    const int* __restrict__ slots, float* __restrict__ rec, int ld_rec, int H, int G, int dk, int dv) {
  extern __shared__ float act[];  // [channels] convolved and activated
  const int t = blockIdx.x;
  const int r = token_req[t];
  const int first = q_start[r];
  const int local = t - first;
  const int C = 2 * G * dk + H * dv;
  const float* tail = state + (size_t)slots[r] * state_stride + tail_off;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int src = local - (taps - 1) + j;
      const float x = src >= 0 ? to_f32<T>(proj[(size_t)(first + src) * ld + c])
                               : tail[(size_t)(src + taps - 1) * C + c];
      acc = fmaf(conv_w[(size_t)c * taps + j], x, acc);
    }
    act[c] = silu_f32(acc);
  }
  __syncthreads();
  float* out = rec + (size_t)t * ld_rec;
  const int lane = threadIdx.x & (TK_WAVE - 1), wave = threadIdx.x / TK_WAVE;
  const int nwaves = blockDim.x / TK_WAVE;
  const float q_scale = 1.0f / sqrtf((float)dk);
  for (int head = wave; head < 2 * G; head += nwaves) {  // q heads, then k heads: unit vectors
    const float* x = act + head * dk;
    float ss = 0.f;
    for (int i = lane; i < dk; i += TK_WAVE) ss = fmaf(x[i], x[i], ss);
    ss = wave_sum(ss);
    float inv = 1.0f / sqrtf(ss + 1e-6f);
    if (head < G) inv *= q_scale;
    for (int i = lane; i < dk; i += TK_WAVE) out[head * dk + i] = x[i] * inv;
  }
  const int v_off = 2 * G * dk, decay_off = v_off + H * dv, beta_off = decay_off + H * dk;
  for (int i = threadIdx.x; i < H * dv; i += blockDim.x) out[v_off + i] = act[v_off + i];
  for (int i = threadIdx.x; i < H * dk; i += blockDim.x) {
    const float rate = expf(a_log[i / dk]);
    out[decay_off + i] = expf(-rate * softplus_f32(a_pre[(size_t)t * H * dk + i] + dt_bias[i]));
  }
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    out[beta_off + i] = sigmoid_f32(to_f32<T>(proj[(size_t)t * ld + col_b + i]));
}

// The convolutions' tails after the step: the last taps - 1 inputs of every request, taken
// from this step's rows and, where the step brought fewer, from the old tail.  A thread a
// (request, channel); it reads all it needs before it writes.
template <typename T>
__global__ void delta_tail_kernel(const T* __restrict__ proj, int ld, int taps, float* __restrict__ state,
                                  size_t state_stride, size_t tail_off, const int* __restrict__ q_start,
                                  const int* __restrict__ slots, int C) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int first = q_start[r], n = q_start[r + 1] - first;
  float* tail = state + (size_t)slots[r] * state_stride + tail_off;
  float keep[DR_MAX_TAPS];
#pragma unroll
  for (int s = 0; s < DR_MAX_TAPS - 1; ++s) {
    if (s < taps - 1) {
      const int src = n - (taps - 1) + s;
      keep[s] = src >= 0 ? to_f32<T>(proj[(size_t)(first + src) * ld + c]) : tail[(size_t)(src + taps - 1) * C + c];
    }
  }
#pragma unroll
  for (int s = 0; s < DR_MAX_TAPS - 1; ++s)
    if (s < taps - 1) tail[(size_t)s * C + c] = keep[s];
}

// --------------------------------------------------------------------------
// The recurrence.  Workgroup (head, request, block of value columns); thread (column, lane):
// the lane holds rows 4 * (lane + DR_LANES * n) + e of its column, n < NQ, e < 4.
// --------------------------------------------------------------------------
template <int NQ>
__global__ __launch_bounds__(NQ > 4 ? 256 : 1024) void delta_rule_kernel(
    const float* __restrict__ rec, int ld_rec, float* __restrict__ state, size_t state_stride,
    const int* __restrict__ q_start, const int* __restrict__ slots, float* __restrict__ o, int H, int G,
    int dk, int dv, int cols) {
  extern __shared__ __align__(16) float stage[];  // [DR_TOKENS][3][dkp] q, k, decay; [DR_TOKENS][cols] v; [DR_TOKENS] beta
  const int h = blockIdx.x, r = blockIdx.y;
  const int col0 = blockIdx.z * cols;
  const int lane = threadIdx.x % DR_LANES;
  const int col = col0 + threadIdx.x / DR_LANES;
  const bool live = col < dv;
  const int dkp = NQ * DR_LANES * 4;  // dk rounded up to what the lanes of a column hold
  const int gk = h / (H / G);
  const int first = q_start[r], last = q_start[r + 1];
  float* s_col = state + (size_t)slots[r] * state_stride + ((size_t)h * dv + (live ? col : 0)) * dk;

  float s[NQ][4];
#pragma unroll
  for (int n = 0; n < NQ; ++n)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = 4 * (lane + DR_LANES * n) + e;
      s[n][e] = (live && i < dk) ? s_col[i] : 0.f;
    }

  float* sq = stage;
  float* sv = stage + DR_TOKENS * 3 * dkp;
  float* sb = sv + DR_TOKENS * cols;
  const int q_off = gk * dk, k_off = G * dk + gk * dk, v_off = 2 * G * dk + h * dv;
  const int g_off = 2 * G * dk + H * dv + h * dk, b_off = 2 * G * dk + H * dv + H * dk + h;

  for (int t0 = first; t0 < last; t0 += DR_TOKENS) {
    const int nt = min(DR_TOKENS, last - t0);
    __syncthreads();  // the chunk before is consumed
    for (int x = threadIdx.x; x < nt * dkp; x += blockDim.x) {
      const int tt = x / dkp, i = x % dkp;
      const float* row = rec + (size_t)(t0 + tt) * ld_rec;
      const bool in = i < dk;
      sq[(tt * 3 + 0) * dkp + i] = in ? row[q_off + i] : 0.f;
      sq[(tt * 3 + 1) * dkp + i] = in ? row[k_off + i] : 0.f;
      sq[(tt * 3 + 2) * dkp + i] = in ? row[g_off + i] : 0.f;
    }
    for (int x = threadIdx.x; x < nt * cols; x += blockDim.x) {
      const int tt = x / cols, c = x % cols;
      sv[x] = (col0 + c < dv) ? rec[(size_t)(t0 + tt) * ld_rec + v_off + col0 + c] : 0.f;
    }
    for (int x = threadIdx.x; x < nt; x += blockDim.x) sb[x] = rec[(size_t)(t0 + x) * ld_rec + b_off];
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float4* q4 = (const float4*)(sq + (tt * 3 + 0) * dkp);
      const float4* k4 = (const float4*)(sq + (tt * 3 + 1) * dkp);
      const float4* g4 = (const float4*)(sq + (tt * 3 + 2) * dkp);
      float kk[NQ][4];
      float dot = 0.f;
#pragma unroll
      for (int n = 0; n < NQ; ++n) {
        const float4 g = g4[lane + DR_LANES * n], k = k4[lane + DR_LANES * n];
        kk[n][0] = k.x; kk[n][1] = k.y; kk[n][2] = k.z; kk[n][3] = k.w;
        s[n][0] *= g.x; s[n][1] *= g.y; s[n][2] *= g.z; s[n][3] *= g.w;
#pragma unroll
        for (int e = 0; e < 4; ++e) dot = fmaf(kk[n][e], s[n][e], dot);
      }
#pragma unroll
      for (int m = 1; m < DR_LANES; m <<= 1) dot += __shfl_xor(dot, m, TK_WAVE);
      const float u = sb[tt] * (sv[tt * cols + threadIdx.x / DR_LANES] - dot);
      float od = 0.f;
#pragma unroll
      for (int n = 0; n < NQ; ++n) {
        const float4 q = q4[lane + DR_LANES * n];
        const float qq[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s[n][e] = fmaf(kk[n][e], u, s[n][e]);
          od = fmaf(qq[e], s[n][e], od);
        }
      }
#pragma unroll
      for (int m = 1; m < DR_LANES; m <<= 1) od += __shfl_xor(od, m, TK_WAVE);
      if (live && lane == 0) o[(size_t)(t0 + tt) * H * dv + (size_t)h * dv + col] = od;
    }
  }
  if (live) {
#pragma unroll
    for (int n = 0; n < NQ; ++n)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * (lane + DR_LANES * n) + e;
        if (i < dk) s_col[i] = s[n][e];
      }
  }
}

// --------------------------------------------------------------------------
// After the recurrence: every head's dv outputs divided by their root mean square, times a
// weight [dv] shared by the heads, times sigmoid(gate); rounded once to T.  A wavefront a
// (token, head).
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ gate,
                                                              const float* __restrict__ w, float eps,
                                                              T* __restrict__ out, long units, int dv) {
  const int lane = threadIdx.x & (TK_WAVE - 1);
  const long unit = (long)blockIdx.x * (blockDim.x / TK_WAVE) + threadIdx.x / TK_WAVE;
  if (unit >= units) return;
  const float* x = o + (size_t)unit * dv;
  const float* g = gate + (size_t)unit * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += TK_WAVE) ss = fmaf(x[i], x[i], ss);
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int i = lane; i < dv; i += TK_WAVE)
    out[(size_t)unit * dv + i] = from_f32<T>(x[i] * rstd * w[i] * sigmoid_f32(g[i]));
}

TK_API int tk_delta_prepare(int dt, const void* proj, int ld, int col_b, const float* a_pre,
                            const float* conv_w, int taps, const float* a_log, const float* dt_bias,
                            float* state, size_t state_stride, size_t tail_off, const int* q_start,
                            const int* token_req, const int* slots, float* rec, int ld_rec, int n_tokens,
                            int n_requests, int H, int G, int dk, int dv, hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && n_requests >= 0 && H > 0 && G > 0 && H % G == 0 && dk > 0 && dv > 0,
             "delta_prepare: bad sizes tokens=%d heads=%d kv heads=%d dk=%d dv=%d", n_tokens, H, G, dk, dv);
  TK_REQUIRE(taps >= 1 && taps <= DR_MAX_TAPS, "delta_prepare: %d taps (1..%d)", taps, DR_MAX_TAPS);
  const int C = 2 * G * dk + H * dv;
  TK_REQUIRE(ld >= C && col_b >= 0 && col_b + H <= ld, "delta_prepare: row stride %d too short", ld);
  TK_REQUIRE(ld_rec >= C + H * dk + H, "delta_prepare: output stride %d too short", ld_rec);
  TK_REQUIRE(tail_off + (size_t)(taps - 1) * C <= state_stride, "delta_prepare: the state row is too short");
  TK_REQUIRE((size_t)C * 4 <= 64 * 1024, "delta_prepare: %d channels do not fit the local memory", C);
  if (n_tokens == 0) return 0;
  const size_t smem = sizeof(float) * (size_t)C;
  if (dt == TK_F32) {
    hipLaunchKernelGGL(delta_prepare_kernel<float>, dim3(n_tokens), dim3(256), smem, stream, (const float*)proj, ld,
                       col_b, a_pre, conv_w, taps, a_log, dt_bias, state, state_stride, tail_off, q_start,
                       token_req, slots, rec, ld_rec, H, G, dk, dv);
  } else {
    hipLaunchKernelGGL(delta_prepare_kernel<bf16_t>, dim3(n_tokens), dim3(256), smem, stream, (const bf16_t*)proj, ld,
                       col_b, a_pre, conv_w, taps, a_log, dt_bias, state, state_stride, tail_off, q_start,
                       token_req, slots, rec, ld_rec, H, G, dk, dv);
  }
  TK_CHECK_LAUNCH("delta_prepare");
  if (taps > 1 && n_requests > 0) {
    TK_REQUIRE(n_requests < 65536, "delta_prepare: too many requests");
    const dim3 grid((C + 255) / 256, n_requests);
    if (dt == TK_F32)
      hipLaunchKernelGGL(delta_tail_kernel<float>, grid, dim3(256), 0, stream, (const float*)proj, ld, taps, state,
                         state_stride, tail_off, q_start, slots, C);
    else
      hipLaunchKernelGGL(delta_tail_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)proj, ld, taps, state,
                         state_stride, tail_off, q_start, slots, C);
    TK_CHECK_LAUNCH("delta_tail");
  }
  return 0;
}

TK_API int tk_delta_rule(const float* rec, int ld_rec, float* state, size_t state_stride, const int* q_start,
                         const int* slots, float* o, int n_requests, int H, int G, int dk, int dv, int cols,
                         hipStream_t stream) {
  TK_REQUIRE(n_requests >= 0 && H > 0 && G > 0 && H % G == 0 && dk > 0 && dv > 0,
             "delta_rule: bad sizes heads=%d kv heads=%d dk=%d dv=%d", H, G, dk, dv);
  TK_REQUIRE(dk <= 512, "delta_rule: key size %d (at most 512)", dk);
  TK_REQUIRE(cols > 0 && cols % (TK_WAVE / DR_LANES) == 0 && cols * DR_LANES <= 1024,
             "delta_rule: %d columns a workgroup", cols);
  TK_REQUIRE(ld_rec >= 2 * G * dk + H * dv + H * dk + H, "delta_rule: input stride %d too short", ld_rec);
  TK_REQUIRE((size_t)H * dv * dk <= state_stride, "delta_rule: the state row is too short");
  TK_REQUIRE(n_requests < 65536, "delta_rule: too many requests");
  if (n_requests == 0) return 0;
  int nq = (dk + DR_LANES * 4 - 1) / (DR_LANES * 4);
  nq = nq <= 2 ? nq : (nq <= 4 ? 4 : (nq <= 8 ? 8 : 16));  // the kernel's instances
  TK_REQUIRE(nq <= 4 || cols * DR_LANES <= 256, "delta_rule: key size %d takes at most %d columns a workgroup", dk,
             256 / DR_LANES);
  const int dkp = nq * DR_LANES * 4;
  const size_t smem = sizeof(float) * ((size_t)DR_TOKENS * 3 * dkp + (size_t)DR_TOKENS * cols + DR_TOKENS);
  const dim3 grid(H, n_requests, (dv + cols - 1) / cols), block(cols * DR_LANES);
#define DR_CASE(NQ)                                                                                       \
  hipLaunchKernelGGL(delta_rule_kernel<NQ>, grid, block, smem, stream, rec, ld_rec, state, state_stride, \
                     q_start, slots, o, H, G, dk, dv, cols)
  if (nq == 1) DR_CASE(1);
  else if (nq == 2) DR_CASE(2);
  else if (nq == 4) DR_CASE(4);
  else if (nq == 8) DR_CASE(8);
  else DR_CASE(16);
#undef DR_CASE
  TK_CHECK_LAUNCH("delta_rule");
  return 0;
}

TK_API int tk_gated_head_norm(int dt, const float* o, const float* gate, const float* w, float eps, void* out,
                              int n_tokens, int H, int dv, hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && H > 0 && dv > 0, "gated_head_norm: bad sizes %d %d %d", n_tokens, H, dv);
  if (n_tokens == 0) return 0;
  const long units = (long)n_tokens * H;
  const long blocks = (units + 3) / 4;
  TK_REQUIRE(blocks < (1l << 31), "gated_head_norm: too many rows");
  if (dt == TK_F32)
    hipLaunchKernelGGL(gated_head_norm_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, o, gate, w, eps,
                       (float*)out, units, dv);
  else
    hipLaunchKernelGGL(gated_head_norm_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, o, gate, w, eps,
                       (bf16_t*)out, units, dv);
  TK_CHECK_LAUNCH("gated_head_norm");
  return 0;
}
