// Mixture of experts: the router (float logits, the `top` largest, softmax over those alone) and the
// activation of the experts' up projections with the routing weights applied. Logits, their order, the
// exponentials and the weights are float whatever the activations' type.
#include "common.h"
#include "reinfer_hip.h"

// ---------------------------------------------------------------------------
// One wave a token: z[e] = sum_i x[t, i] * Wr[e, i] (float; lanes split i and add in a fixed order), then
// `top` rounds of a wave-wide maximum (ties go to the lower expert), then p_j = exp(z_j - z_0) / sum.
// ids[t, j] and weights[t, j] come out in falling order of z.
// ---------------------------------------------------------------------------
template <typename TA>
__global__ void moe_route_kernel(const TA* __restrict__ x, int ldx, const float* __restrict__ Wr, int E, int width,
                                 int top, int* __restrict__ ids, float* __restrict__ weights) {
  extern __shared__ float z[];           // [E]
  const int t = blockIdx.x;
  const int lane = threadIdx.x;
  const TA* row = x + (size_t)t * ldx;
  for (int e = 0; e < E; ++e) {
    const float* w = Wr + (size_t)e * width;
    float s = 0.f;
    for (int i = lane; i < width; i += RA_WAVE) s += to_f32(row[i]) * w[i];
    s = wave_sum(s);
    if (lane == 0) z[e] = s;
  }
  __syncthreads();
  float z0 = 0.f, denom = 0.f, mine = 0.f;
  int mine_id = 0;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += RA_WAVE) {
      const float v = z[e];
      if (v > best) { best = v; at = e; }         // ascending e: the first of equals stays
    }
#pragma unroll
    for (int m = RA_WAVE / 2; m > 0; m >>= 1) {
      const float ob = __shfl_xor(best, m, RA_WAVE);
      const int oa = __shfl_xor(at, m, RA_WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (j == 0) z0 = best;
    const float p = expf(best - z0);
    denom += p;
    if (lane == j) { mine = p; mine_id = at; }    // lane j keeps the j-th choice (top <= 64)
    __syncthreads();
    if (lane == 0 && at < E) z[at] = -INFINITY;
    __syncthreads();
  }
  if (lane < top) {
    weights[(size_t)t * top + lane] = mine / denom;
    ids[(size_t)t * top + lane] = mine_id;
  }
}

extern "C" int ra_moe_route(const void* x, int act_dtype, int ldx, const float* router, int experts, int width,
                            int top, int* ids, float* weights, int n_tokens, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && experts > 0 && width > 0, "moe_route: %d tokens, %d experts, width %d", n_tokens, experts, width);
  RA_CHECK(top > 0 && top <= experts && top <= RA_WAVE, "moe_route: %d of %d experts (at most 64 chosen)", top, experts);
  RA_CHECK(ldx >= width, "moe_route: rows of %d for width %d", ldx, width);
  const size_t lds = (size_t)experts * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "moe_route: %d experts", experts);
  if (act_dtype == RA_F32)
    moe_route_kernel<float><<<n_tokens, RA_WAVE, lds, stream>>>((const float*)x, ldx, router, experts, width, top, ids, weights);
  else if (act_dtype == RA_BF16)
    moe_route_kernel<bf16_t><<<n_tokens, RA_WAVE, lds, stream>>>((const bf16_t*)x, ldx, router, experts, width, top, ids, weights);
  else
    return ra_fail("moe_route: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_route");
  return 0;
}

// ---------------------------------------------------------------------------
// Experts side by side: up[t, e * ff + j] is expert e's up projection of token t. act[t, e * ff + j] =
// p(t, e) * relu(up)^2 for the chosen experts, 0 for the others, so that one product with the down
// projections laid side by side, [width, E * ff], is the weighted sum of the chosen experts' outputs.
// ---------------------------------------------------------------------------
template <typename TA>
__global__ void moe_relu2_scale_kernel(const TA* __restrict__ up, TA* __restrict__ act, const int* __restrict__ ids,
                                       const float* __restrict__ weights, int top, int E, int ff) {
  extern __shared__ float gate[];        // [E]
  const int t = blockIdx.y;
  for (int e = threadIdx.x; e < E; e += blockDim.x) gate[e] = 0.f;
  __syncthreads();
  for (int j = threadIdx.x; j < top; j += blockDim.x) gate[ids[(size_t)t * top + j]] = weights[(size_t)t * top + j];
  __syncthreads();
  const int n = E * ff;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const float g = gate[i / ff];
    float v = 0.f;
    if (g != 0.f) {
      const float u = fmaxf(to_f32(up[(size_t)t * n + i]), 0.f);
      v = g * (u * u);
    }
    act[(size_t)t * n + i] = from_f32<TA>(v);
  }
}

extern "C" int ra_moe_relu2_scale(const void* up, void* act, int act_dtype, const int* ids, const float* weights,
                                  int top, int experts, int ff, int n_tokens, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && experts > 0 && ff > 0 && top > 0 && top <= experts,
           "moe_relu2_scale: %d tokens, %d of %d experts of %d", n_tokens, top, experts, ff);
  RA_CHECK(n_tokens <= 65535, "moe_relu2_scale: %d tokens in one launch (max 65535)", n_tokens);
  const size_t lds = (size_t)experts * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "moe_relu2_scale: %d experts", experts);
  dim3 grid((experts * ff + 255) / 256, n_tokens);
  if (act_dtype == RA_F32)
    moe_relu2_scale_kernel<float><<<grid, 256, lds, stream>>>((const float*)up, (float*)act, ids, weights, top, experts, ff);
  else if (act_dtype == RA_BF16)
    moe_relu2_scale_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)up, (bf16_t*)act, ids, weights, top, experts, ff);
  else
    return ra_fail("moe_relu2_scale: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_relu2_scale");
  return 0;
}
