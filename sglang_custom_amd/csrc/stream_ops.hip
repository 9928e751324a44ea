// Kernels around a 32-bit residual stream whose sequences carry state from step to step:
//   * token + hashed-bigram embedding (the previous token of a sequence is state),
//   * weight-only layer norm fused with the token shift (the previous token's normed row is state),
//   * the commit of a step's new state rows,
//   * tanh-GELU-and-mul, and the sigmoid-gated residual update.
// Every reduction, normalisation, gate and the residual sum run in fp32 whatever the activation dtype T is;
// T only names what the GEMMs around these kernels read and write.
//
// Batch description shared by the kernels (all device pointers):
//   tok_req[t]    index b of token t's sequence in the batch        (null: b = t, every token is its own segment)
//   seg_start[b]  first token of b's segment in the flat token list (null with tok_req)
//   seg_len[b]    number of tokens of b in this step
//   positions[t]  position of token t in its sequence
//   req_pool_indices[b] -> req_to_state[.] = the sequence's state slot
#include "common.cuh"

#include <algorithm>

namespace mi355 {
namespace {

struct Seg {
  int b;
  bool first, last;
};
__device__ __forceinline__ Seg segment_of(int64_t t, const int32_t* tok_req, const int32_t* seg_start, const int32_t* seg_len) {
  Seg s;
  if (tok_req == nullptr) {
    s.b = (int)t;
    s.first = s.last = true;
  } else {
    s.b = tok_req[t];
    const int64_t t0 = seg_start[s.b];
    s.first = t == t0;
    s.last = t == t0 + seg_len[s.b] - 1;
  }
  return s;
}

// (x - mean) / sqrt(var + eps) of one row into buf (LDS, D floats); var = mean of squared deviations.  Every thread
// touches the same elements in all three passes, so buf needs no barrier of its own.  W = 4: four floats per access
// (D a multiple of 4, rows 16-byte aligned).
template <int W>
__device__ __forceinline__ void ln_row(float* buf, const float* __restrict__ x, int64_t D, float eps, float* red) {
  float s = 0.f;
  for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
    if constexpr (W == 4) {
      const float4 v = *reinterpret_cast<const float4*>(x + i);
      *reinterpret_cast<float4*>(buf + i) = v;
      s += (v.x + v.y) + (v.z + v.w);
    } else {
      const float v = x[i];
      buf[i] = v;
      s += v;
    }
  }
  const float mean = block_sum(s, red) / (float)D;
  float q = 0.f;
  for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
#pragma unroll
    for (int k = 0; k < W; ++k) {
      const float d = buf[i + k] - mean;
      q += d * d;
    }
  }
  const float var = block_sum(q, red) / (float)D;
  const float inv = 1.0f / sqrtf(var + eps);
  for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
#pragma unroll
    for (int k = 0; k < W; ++k) buf[i + k] = (buf[i + k] - mean) * inv;
  }
}

// One workgroup per token.  h = LN(x[t]) * w;  with `mu`: hs = h + (h_prev - h) * mu, where h_prev is the same
// quantity of the previous token: zero at position 0, the state row when t opens its segment, else recomputed from
// x[t - 1].  The last token of every segment leaves its fp32 h in h_last[b] for the commit kernel.
template <typename T, int W>
__global__ __launch_bounds__(256) void layernorm_shift_kernel(
    T* __restrict__ h_out, T* __restrict__ hs_out, float* __restrict__ h_last, const float* __restrict__ x,
    const T* __restrict__ w, const T* __restrict__ mu, const float* __restrict__ state, const int32_t* __restrict__ req_to_state,
    const int64_t* __restrict__ req_pool_indices, const int32_t* __restrict__ tok_req, const int32_t* __restrict__ seg_start,
    const int32_t* __restrict__ seg_len, const int64_t* __restrict__ positions, int64_t D, float eps) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  __shared__ float red[16];
  float* cur = sm;
  float* prv = sm + D;
  const int64_t t = blockIdx.x;
  const int64_t i0 = W * threadIdx.x, step = W * blockDim.x;
  ln_row<W>(cur, x + t * D, D, eps, red);
  if (mu == nullptr) {
    for (int64_t i = i0; i < D; i += step) {
      Vec<T, W> o;
#pragma unroll
      for (int k = 0; k < W; ++k) o.v[k] = from_f32<T>(cur[i + k] * to_f32(w[i + k]));
      stvec<T, W>(h_out + t * D + i, o);
    }
    return;
  }
  const Seg sg = segment_of(t, tok_req, seg_start, seg_len);
  const int64_t pos = positions[t];
  if (pos == 0) {
    for (int64_t i = i0; i < D; i += step)
#pragma unroll
      for (int k = 0; k < W; ++k) prv[i + k] = 0.f;
  } else if (sg.first) {
    const float* srow = state + (int64_t)req_to_state[req_pool_indices[sg.b]] * D;
    for (int64_t i = i0; i < D; i += step)
#pragma unroll
      for (int k = 0; k < W; ++k) prv[i + k] = srow[i + k];
  } else {
    ln_row<W>(prv, x + (t - 1) * D, D, eps, red);
    for (int64_t i = i0; i < D; i += step)
#pragma unroll
      for (int k = 0; k < W; ++k) prv[i + k] *= to_f32(w[i + k]);
  }
  const bool keep = sg.last && h_last != nullptr;
  for (int64_t i = i0; i < D; i += step) {
    Vec<T, W> ho, so;
#pragma unroll
    for (int k = 0; k < W; ++k) {
      const float h = cur[i + k] * to_f32(w[i + k]);
      ho.v[k] = from_f32<T>(h);
      so.v[k] = from_f32<T>(h + (prv[i + k] - h) * to_f32(mu[i + k]));
      if (keep) h_last[(int64_t)sg.b * D + i + k] = h;
    }
    stvec<T, W>(h_out + t * D + i, ho);
    stvec<T, W>(hs_out + t * D + i, so);
  }
}

// x[t] = table[id] * scale + bigram[(prev * mul_prev + id * mul_cur) mod buckets]; row `buckets` at position 0.
template <typename T>
__global__ __launch_bounds__(256) void bigram_embedding_kernel(
    float* __restrict__ x, const int64_t* __restrict__ ids, const T* __restrict__ table, const T* __restrict__ bigram,
    const int32_t* __restrict__ prev_token, const int32_t* __restrict__ req_to_state, const int64_t* __restrict__ req_pool_indices,
    const int32_t* __restrict__ tok_req, const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
    const int64_t* __restrict__ positions, int64_t D, int64_t vocab, float scale, int64_t mul_prev, int64_t mul_cur,
    int64_t buckets) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const Seg sg = segment_of(t, tok_req, seg_start, seg_len);
  int64_t row = buckets;
  if (positions[t] != 0) {
    int64_t prev;
    if (sg.first)
      prev = prev_token[req_to_state[req_pool_indices[sg.b]]];
    else
      prev = ids[t - 1];
    row = (prev * mul_prev + id * mul_cur) % buckets;
    if (row < 0) row += buckets;
  }
  const T* e = table + id * D;
  const T* g = bigram + row * D;
  for (int64_t i = threadIdx.x; i < D; i += blockDim.x) x[t * D + i] = to_f32(e[i]) * scale + to_f32(g[i]);
}

// grid (B, L): state[l][slot(b)] = h_last[l][b]; layer 0's workgroups also store the segment's last token id.
__global__ __launch_bounds__(256) void commit_state_kernel(
    float* __restrict__ state, int32_t* __restrict__ prev_token, const float* __restrict__ h_last, const int64_t* __restrict__ ids,
    const int32_t* __restrict__ req_to_state, const int64_t* __restrict__ req_pool_indices, const int32_t* __restrict__ seg_start,
    const int32_t* __restrict__ seg_len, int64_t B, int64_t D, int64_t state_layer_stride) {
  const int64_t b = blockIdx.x, l = blockIdx.y;
  const int64_t slot = req_to_state[req_pool_indices[b]];
  const float* src = h_last + (l * B + b) * D;
  float* dst = state + l * state_layer_stride + slot * D;
  for (int64_t i = threadIdx.x; i < D; i += blockDim.x) dst[i] = src[i];
  if (l == 0 && threadIdx.x == 0 && prev_token != nullptr) {
    const int64_t last = seg_start ? (int64_t)seg_start[b] + seg_len[b] - 1 : b;
    prev_token[slot] = (int32_t)ids[last];
  }
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

// out[t][i] = gelu_tanh(gate[t][i]) * up[t][i], 16 bytes of each operand per thread (d and the row stride multiples of the
// vector length, pointers 16-byte aligned)
template <typename T>
__global__ __launch_bounds__(256) void gelu_tanh_and_mul_vec_kernel(T* __restrict__ out, const T* __restrict__ gate, const T* __restrict__ up,
                                                                   int64_t rows, int64_t d, int64_t in_stride) {
  constexpr int VE = V16<T>::n;
  const int64_t per_row = d / VE, n = rows * per_row;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / per_row, i = (idx - r * per_row) * VE;
    const Vec<T, VE> g = ldvec<T, VE>(gate + r * in_stride + i), u = ldvec<T, VE>(up + r * in_stride + i);
    Vec<T, VE> o;
#pragma unroll
    for (int j = 0; j < VE; ++j) o.v[j] = from_f32<T>(gelu_tanh_f(to_f32(g.v[j])) * to_f32(u.v[j]));
    stvec<T, VE>(out + r * d + i, o);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_tanh_and_mul_kernel(T* __restrict__ out, const T* __restrict__ gate, const T* __restrict__ up,
                                                               int64_t rows, int64_t d, int64_t in_stride) {
  const int64_t n = rows * d;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / d, i = idx - r * d;
    out[idx] = from_f32<T>(gelu_tanh_f(to_f32(gate[r * in_stride + i])) * to_f32(up[r * in_stride + i]));
  }
}

// x[t][i] += sigmoid(g1[t][i] + b1[i]) * y1[t][i] (+ the same with g2, b2, y2 when y2 is given)
template <typename T>
__global__ __launch_bounds__(256) void gated_residual_kernel(
    float* __restrict__ x, const T* __restrict__ g1, const T* __restrict__ b1, const T* __restrict__ y1, const T* __restrict__ g2,
    const T* __restrict__ b2, const T* __restrict__ y2, int64_t rows, int64_t d, int64_t g_stride, int64_t y1_stride,
    int64_t y2_stride) {
  const int64_t n = rows * d;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / d, i = idx - r * d;
    float add = sigmoid_f(to_f32(g1[r * g_stride + i]) + to_f32(b1[i])) * to_f32(y1[r * y1_stride + i]);
    if (y2 != nullptr) add += sigmoid_f(to_f32(g2[r * g_stride + i]) + to_f32(b2[i])) * to_f32(y2[r * y2_stride + i]);
    x[idx] += add;
  }
}

}  // namespace
}  // namespace mi355

using namespace mi355;

int mi355_layernorm_shift(void* h_out, void* hs_out, float* h_last, const float* x, const void* weight, const void* shift,
                          const float* state, const int32_t* req_to_state, const int64_t* req_pool_indices,
                          const int32_t* tok_req, const int32_t* seg_start, const int32_t* seg_len, const int64_t* positions,
                          int64_t tokens, int64_t hidden, float eps, int dtype, void* stream) {
  MI355_REQUIRE(h_out && x && weight, MI355_ERR_INVALID, "layernorm_shift: null pointer");
  MI355_REQUIRE(tokens >= 0 && hidden > 0 && hidden <= 16384, MI355_ERR_INVALID, "layernorm_shift: bad shape");
  MI355_REQUIRE(shift == nullptr || (hs_out && state && req_to_state && req_pool_indices && positions), MI355_ERR_INVALID,
                "layernorm_shift: the token shift needs hs_out, the state rows, the slot map and positions");
  MI355_REQUIRE((tok_req == nullptr) == (seg_start == nullptr) && (tok_req == nullptr) == (seg_len == nullptr), MI355_ERR_INVALID,
                "layernorm_shift: tok_req, seg_start and seg_len come together");
  if (tokens == 0) return MI355_OK;
  const size_t lds = (size_t)hidden * 2 * sizeof(float);
  MI355_DISPATCH_DTYPE(dtype, "layernorm_shift", {
    const bool wide = hidden % 4 == 0 && aligned16(x) && aligned16(h_out) && (!hs_out || aligned16(hs_out)) &&
                      (!state || aligned16(state));
    auto kern = wide ? layernorm_shift_kernel<T, 4> : layernorm_shift_kernel<T, 1>;
    if (lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, dim3((unsigned)tokens), dim3(256), lds, (hipStream_t)stream, (T*)h_out, (T*)hs_out, h_last, x,
                       (const T*)weight, (const T*)shift, state, req_to_state, req_pool_indices, tok_req, seg_start, seg_len,
                       positions, hidden, eps);
  });
  MI355_CHECK_LAUNCH("layernorm_shift");
  return MI355_OK;
}

int mi355_bigram_embedding(float* x, const int64_t* ids, const void* table, const void* bigram, const int32_t* prev_token,
                           const int32_t* req_to_state, const int64_t* req_pool_indices, const int32_t* tok_req,
                           const int32_t* seg_start, const int32_t* seg_len, const int64_t* positions, int64_t tokens,
                           int64_t hidden, int64_t vocab, float scale, int64_t mul_prev, int64_t mul_cur, int64_t buckets,
                           int dtype, void* stream) {
  MI355_REQUIRE(x && ids && table && bigram && prev_token && req_to_state && req_pool_indices && positions, MI355_ERR_INVALID,
                "bigram_embedding: null pointer");
  MI355_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0 && buckets > 0, MI355_ERR_INVALID, "bigram_embedding: bad shape");
  MI355_REQUIRE((tok_req == nullptr) == (seg_start == nullptr) && (tok_req == nullptr) == (seg_len == nullptr), MI355_ERR_INVALID,
                "bigram_embedding: tok_req, seg_start and seg_len come together");
  if (tokens == 0) return MI355_OK;
  MI355_DISPATCH_DTYPE(dtype, "bigram_embedding", {
    hipLaunchKernelGGL((bigram_embedding_kernel<T>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, x, ids,
                       (const T*)table, (const T*)bigram, prev_token, req_to_state, req_pool_indices, tok_req, seg_start, seg_len,
                       positions, hidden, vocab, scale, mul_prev, mul_cur, buckets);
  });
  MI355_CHECK_LAUNCH("bigram_embedding");
  return MI355_OK;
}

int mi355_commit_sequence_state(float* state, int32_t* prev_token, const float* h_last, const int64_t* ids,
                                const int32_t* req_to_state, const int64_t* req_pool_indices, const int32_t* seg_start,
                                const int32_t* seg_len, int64_t batch, int64_t layers, int64_t hidden, int64_t state_layer_stride,
                                void* stream) {
  MI355_REQUIRE(state && h_last && ids && req_to_state && req_pool_indices, MI355_ERR_INVALID, "commit_sequence_state: null pointer");
  MI355_REQUIRE(batch >= 0 && layers > 0 && layers < 65536 && hidden > 0, MI355_ERR_INVALID, "commit_sequence_state: bad shape");
  MI355_REQUIRE((seg_start == nullptr) == (seg_len == nullptr), MI355_ERR_INVALID, "commit_sequence_state: seg_start and seg_len come together");
  if (batch == 0) return MI355_OK;
  hipLaunchKernelGGL(commit_state_kernel, dim3((unsigned)batch, (unsigned)layers), dim3(256), 0, (hipStream_t)stream, state,
                     prev_token, h_last, ids, req_to_state, req_pool_indices, seg_start, seg_len, batch, hidden, state_layer_stride);
  MI355_CHECK_LAUNCH("commit_sequence_state");
  return MI355_OK;
}

int mi355_gelu_tanh_and_mul(void* out, const void* gate, const void* up, int64_t rows, int64_t d, int64_t in_stride, int dtype,
                            void* stream) {
  MI355_REQUIRE(out && gate && up, MI355_ERR_INVALID, "gelu_tanh_and_mul: null pointer");
  MI355_REQUIRE(rows >= 0 && d > 0 && in_stride >= d, MI355_ERR_INVALID, "gelu_tanh_and_mul: bad shape");
  if (rows == 0) return MI355_OK;
  const int grid = (int)std::min<int64_t>((rows * d + 255) / 256, 256 * 16);
  MI355_DISPATCH_DTYPE(dtype, "gelu_tanh_and_mul", {
    constexpr int VE = V16<T>::n;
    if (d % VE == 0 && in_stride % VE == 0 && aligned16(out) && aligned16(gate) && aligned16(up)) {
      const int vgrid = (int)std::min<int64_t>((rows * (d / VE) + 255) / 256, 256 * 16);
      hipLaunchKernelGGL((gelu_tanh_and_mul_vec_kernel<T>), dim3(vgrid), dim3(256), 0, (hipStream_t)stream, (T*)out, (const T*)gate,
                         (const T*)up, rows, d, in_stride);
    } else {
      hipLaunchKernelGGL((gelu_tanh_and_mul_kernel<T>), dim3(grid), dim3(256), 0, (hipStream_t)stream, (T*)out, (const T*)gate,
                         (const T*)up, rows, d, in_stride);
    }
  });
  MI355_CHECK_LAUNCH("gelu_tanh_and_mul");
  return MI355_OK;
}

int mi355_gated_residual_add(float* x, const void* g1, const void* b1, const void* y1, const void* g2, const void* b2,
                             const void* y2, int64_t rows, int64_t d, int64_t g_stride, int64_t y1_stride, int64_t y2_stride,
                             int dtype, void* stream) {
  MI355_REQUIRE(x && g1 && b1 && y1, MI355_ERR_INVALID, "gated_residual_add: null pointer");
  MI355_REQUIRE(y2 == nullptr || (g2 && b2), MI355_ERR_INVALID, "gated_residual_add: the second branch needs its gate and bias");
  MI355_REQUIRE(rows >= 0 && d > 0, MI355_ERR_INVALID, "gated_residual_add: bad shape");
  if (rows == 0) return MI355_OK;
  const int grid = (int)std::min<int64_t>((rows * d + 255) / 256, 256 * 16);
  MI355_DISPATCH_DTYPE(dtype, "gated_residual_add", {
    hipLaunchKernelGGL((gated_residual_kernel<T>), dim3(grid), dim3(256), 0, (hipStream_t)stream, x, (const T*)g1, (const T*)b1,
                       (const T*)y1, (const T*)g2, (const T*)b2, (const T*)y2, rows, d, g_stride, y1_stride, y2_stride);
  });
  MI355_CHECK_LAUNCH("gated_residual_add");
  return MI355_OK;
}
