// Mixture of experts: the router's choice (the `top` largest float logits, softmax over those alone) and the
// activation of the experts' up projections with the routing weights applied. Logits, their order, the
// exponentials and the weights are float whatever the activations' type.
#include "common.h"
#include "reinfer_hip.h"

// ---------------------------------------------------------------------------
// One wave a token: its float router logits z[0..E) (a product made them) go to LDS, then `top` rounds of a
// wave-wide maximum (ties go to the lower expert), then p_j = exp(z_j - z_0) / sum over the chosen.
// ids[t, j] and weights[t, j] come out in falling order of z.
// ---------------------------------------------------------------------------
#define MOE_TOPK_WAVES 4
__global__ void moe_topk_kernel(const float* __restrict__ logits, int ld, int E, int top, int* __restrict__ ids,
                                float* __restrict__ weights, int T) {
  extern __shared__ float zs[];          // [MOE_TOPK_WAVES][E]
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int t = blockIdx.x * MOE_TOPK_WAVES + wave;
  if (t >= T) return;                    // whole waves leave; no workgroup barrier below
  float* z = zs + (size_t)wave * E;
  for (int e = lane; e < E; e += RA_WAVE) z[e] = logits[(size_t)t * ld + e];
  float z0 = 0.f, denom = 0.f, mine = 0.f;
  int mine_id = 0;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += RA_WAVE) {      // a lane reads back only what it wrote itself
      const float v = z[e];
      if (at == 0x7fffffff || v > best) { best = v; at = e; }       // ascending e: the first of equals stays
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
    if (at < E && (at & (RA_WAVE - 1)) == lane) z[at] = -INFINITY;   // taken: its own lane strikes it
  }
  if (lane < top) {
    weights[(size_t)t * top + lane] = mine / denom;
    ids[(size_t)t * top + lane] = mine_id;
  }
}

extern "C" int ra_moe_topk(const float* logits, int ld, int experts, int top, int* ids, float* weights,
                           int n_tokens, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && experts > 0, "moe_topk: %d tokens, %d experts", n_tokens, experts);
  RA_CHECK(top > 0 && top <= experts && top <= RA_WAVE, "moe_topk: %d of %d experts (at most 64 chosen)", top, experts);
  RA_CHECK(ld >= experts, "moe_topk: rows of %d for %d experts", ld, experts);
  const size_t lds = (size_t)MOE_TOPK_WAVES * experts * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "moe_topk: %d experts", experts);
  const int groups = (n_tokens + MOE_TOPK_WAVES - 1) / MOE_TOPK_WAVES;
  moe_topk_kernel<<<groups, MOE_TOPK_WAVES * RA_WAVE, lds, stream>>>(logits, ld, experts, top, ids, weights, n_tokens);
  RA_LAUNCH_CHECK("moe_topk");
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

// the same, eight bfloat16 columns a thread (ff a multiple of 8: the eight lie in one expert)
__global__ void moe_relu2_scale_x8_kernel(const bf16_t* __restrict__ up, bf16_t* __restrict__ act,
                                          const int* __restrict__ ids, const float* __restrict__ weights, int top,
                                          int E, int ff) {
  extern __shared__ float gate[];        // [E]
  const int t = blockIdx.y;
  for (int e = threadIdx.x; e < E; e += blockDim.x) gate[e] = 0.f;
  __syncthreads();
  for (int j = threadIdx.x; j < top; j += blockDim.x) gate[ids[(size_t)t * top + j]] = weights[(size_t)t * top + j];
  __syncthreads();
  const int n = E * ff;
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i < n) {
    const float g = gate[i / ff];
    bf16x8_t o = {0, 0, 0, 0, 0, 0, 0, 0};
    if (g != 0.f) {
      const bf16x8_t u = *(const bf16x8_t*)(up + (size_t)t * n + i);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float v = fmaxf((float)u[k], 0.f);
        o[k] = (bf16_t)(g * (v * v));
      }
    }
    *(bf16x8_t*)(act + (size_t)t * n + i) = o;
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
  if (act_dtype == RA_BF16 && ff % 8 == 0 && ((uintptr_t)up % 16) == 0 && ((uintptr_t)act % 16) == 0) {
    dim3 grid8((experts * ff / 8 + 255) / 256, n_tokens);
    moe_relu2_scale_x8_kernel<<<grid8, 256, lds, stream>>>((const bf16_t*)up, (bf16_t*)act, ids, weights, top, experts, ff);
  } else if (act_dtype == RA_F32)
    moe_relu2_scale_kernel<float><<<grid, 256, lds, stream>>>((const float*)up, (float*)act, ids, weights, top, experts, ff);
  else if (act_dtype == RA_BF16)
    moe_relu2_scale_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)up, (bf16_t*)act, ids, weights, top, experts, ff);
  else
    return ra_fail("moe_relu2_scale: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_relu2_scale");
  return 0;
}
