// Row kernels around the residual stream that some architectures add to the plain embedding and head:
// rows of a hashed token-pair table added to the embedding (the previous token of a request is kept in a
// per-request state word), vectors and a saved copy of the stream added before a group of layers, and a
// tanh cap on the logits. The stream and every sum are float.
#include "common.h"
#include "reinfer_hip.h"

// ---------------------------------------------------------------------------
// resid[t, :] += table[row(t), :], row(t) = (prev(t) * mul_prev + id(t) * mul_cur) mod buckets, or row
// `buckets` (the table's last) for a request's first token. prev(t) is the token before t in the step, or,
// for the first token of a request's portion, the word that the request's state slot holds. The thread that
// reads that word is also the one that writes the portion's last token back into it, so nothing races;
// rows with state slot -1 (padding of a captured step) read and write no state.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void pair_hash_add_kernel(float* __restrict__ resid, const T* __restrict__ table,
                                     const int* __restrict__ ids, const int* __restrict__ positions,
                                     const int* __restrict__ seq_of_token, const int* __restrict__ cu_tokens,
                                     const int* __restrict__ state_slots, int* __restrict__ last_token,
                                     int buckets, long long mul_prev, long long mul_cur, int h) {
  const int t = blockIdx.x;
  __shared__ int row_s;
  if (threadIdx.x == 0) {
    const int seq = seq_of_token[t];
    const int first = cu_tokens[seq];
    const int slot = state_slots[seq];
    const int pos = positions[t];
    int prev = -1;
    if (t != first) {
      prev = ids[t - 1];
    } else {
      if (pos > 0 && slot >= 0) prev = last_token[slot];
      if (slot >= 0) last_token[slot] = ids[cu_tokens[seq + 1] - 1];
    }
    int row = buckets;
    if (pos > 0 && prev >= 0) {
      long long v = ((long long)prev * mul_prev + (long long)ids[t] * mul_cur) % (long long)buckets;
      if (v < 0) v += buckets;
      row = (int)v;
    }
    row_s = row;
  }
  __syncthreads();
  const T* src = table + (size_t)row_s * h;
  float* o = resid + (size_t)t * h;
  for (int i = threadIdx.x; i < h; i += blockDim.x) o[i] += to_f32(src[i]);
}

extern "C" int ra_pair_hash_add(float* resid, const void* table, int table_dtype, const int* ids,
                                const int* positions, const int* seq_of_token, const int* cu_tokens,
                                const int* state_slots, int* last_token, int buckets, long long mul_prev,
                                long long mul_cur, int n_tokens, int hidden, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && hidden > 0 && buckets > 0, "pair_hash_add: %d tokens, width %d, %d buckets", n_tokens,
           hidden, buckets);
  if (table_dtype == RA_F32)
    pair_hash_add_kernel<float><<<n_tokens, 256, 0, stream>>>(resid, (const float*)table, ids, positions,
                                                              seq_of_token, cu_tokens, state_slots, last_token,
                                                              buckets, mul_prev, mul_cur, hidden);
  else if (table_dtype == RA_BF16)
    pair_hash_add_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(resid, (const bf16_t*)table, ids, positions,
                                                               seq_of_token, cu_tokens, state_slots, last_token,
                                                               buckets, mul_prev, mul_cur, hidden);
  else
    return ra_fail("pair_hash_add: unknown dtype tag %d", table_dtype);
  RA_LAUNCH_CHECK("pair_hash_add");
  return 0;
}

// ---------------------------------------------------------------------------
// resid[t, :] += delta_scale * delta[t, :] + other[t, :] + vec[:]   (each addend optional)
// ---------------------------------------------------------------------------
template <typename TD, typename TV>
__global__ void stream_add_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                  const float* __restrict__ other, const TV* __restrict__ vec, int h,
                                  float dscale) {
  const size_t base = (size_t)blockIdx.x * h;
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    float v = resid[base + i];
    if (delta) v += dscale * to_f32(delta[base + i]);
    if (other) v += other[base + i];
    if (vec) v += to_f32(vec[i]);
    resid[base + i] = v;
  }
}

extern "C" int ra_stream_add(float* resid, const void* delta, int delta_dtype, const float* other, const void* vec,
                             int vec_dtype, int n_tokens, int hidden, float delta_scale, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && hidden > 0, "stream_add: empty input (%d tokens, width %d)", n_tokens, hidden);
#define RA_SA(TD, TV)                                                                                    \
  stream_add_kernel<TD, TV><<<n_tokens, 256, 0, stream>>>(resid, (const TD*)delta, other, (const TV*)vec, hidden, delta_scale)
  if (delta_dtype == RA_F32 && vec_dtype == RA_F32) RA_SA(float, float);
  else if (delta_dtype == RA_F32 && vec_dtype == RA_BF16) RA_SA(float, bf16_t);
  else if (delta_dtype == RA_BF16 && vec_dtype == RA_F32) RA_SA(bf16_t, float);
  else if (delta_dtype == RA_BF16 && vec_dtype == RA_BF16) RA_SA(bf16_t, bf16_t);
  else return ra_fail("stream_add: unknown dtype tags %d, %d", delta_dtype, vec_dtype);
#undef RA_SA
  RA_LAUNCH_CHECK("stream_add");
  return 0;
}

// ---------------------------------------------------------------------------
// logits <- cap * tanh(logits / cap), in place, rows of `vocab` floats `row_stride` apart
// ---------------------------------------------------------------------------
__global__ void tanh_cap_kernel(float* __restrict__ logits, int vocab, int row_stride, float cap) {
  float* row = logits + (size_t)blockIdx.y * row_stride;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < vocab) row[i] = cap * tanhf(row[i] / cap);
}

extern "C" int ra_tanh_cap(float* logits, int n_rows, int vocab, int row_stride, float cap, hipStream_t stream) {
  RA_CHECK(n_rows > 0 && vocab > 0 && row_stride >= vocab, "tanh_cap: %d rows of %d (stride %d)", n_rows, vocab,
           row_stride);
  RA_CHECK(cap > 0.f, "tanh_cap: the cap must be positive");
  RA_CHECK(n_rows <= 65535, "tanh_cap: %d rows in one launch (max 65535)", n_rows);
  dim3 grid((vocab + 255) / 256, n_rows);
  tanh_cap_kernel<<<grid, 256, 0, stream>>>(logits, vocab, row_stride, cap);
  RA_LAUNCH_CHECK("tanh_cap");
  return 0;
}
