// Sliding-window attention over a latent KV cache, with a learned sink in the softmax denominator.
//
// The cache holds one row per token and layer: [ c (rank features) | k_r (rope features, already rotated) ].  In the
// absorbed form every head h attends the same rows: score(t, j) = (qa[t,h] . c[j] + rot(qr[t,h]) . k_r[j]) * scale
// with qa = q_nope W_uk[h], and the result per head is sum_j p(t, j) c[j] (the caller applies W_uv[h]).  Query at
// position p sees key j iff 0 <= p - j < window.  softmax: p(t, j) = exp(s_j - m) / (sum_j exp(s_j - m) + exp(sink_h - m));
// the sink has no value row, so the running (max, sum) pair simply starts at (sink_h, 1).
//
//   mi355_latent_norms_rope_write   the step before it: both latent RMS norms of the "a" projection's row, the
//                                   rotation of the shared rope key and the write of the cache row
//   mi355_latent_window_attention   prefill portions and decode steps alike: a workgroup takes a run of consecutive
//                                   tokens of one sequence x a group of heads and walks the window's cache rows in
//                                   LDS tiles; all arithmetic on scores, weights and sums is fp32
#include "common.cuh"

#include <algorithm>

namespace mi355 {
namespace {

// ------------------------------------------------------------------------------------------ latent norms + rope + cache write
// One workgroup per token.  a[t] = [ q latent (q_rank) | kv latent (rank) | rope key (dr) | ... ].
template <typename T>
__global__ __launch_bounds__(256) void latent_norms_rope_write_kernel(
    T* __restrict__ cq, T* __restrict__ cache, const T* __restrict__ a, const T* __restrict__ wq, const T* __restrict__ wkv,
    const int64_t* __restrict__ positions, const int64_t* __restrict__ loc, const float* __restrict__ inv_freq, int64_t a_stride,
    int q_rank, int rank, int dr, int rot_dims, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const T* row = a + t * a_stride;
  float s = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
    const float v = to_f32(row[i]);
    s += v * v;
  }
  const float inv_q = 1.0f / sqrtf(block_sum(s, red) / (float)q_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) cq[t * q_rank + i] = from_f32<T>(to_f32(row[i]) * inv_q * to_f32(wq[i]));
  s = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = to_f32(row[q_rank + i]);
    s += v * v;
  }
  const float inv_kv = 1.0f / sqrtf(block_sum(s, red) / (float)rank + eps);
  T* dst = cache + loc[t] * (int64_t)(rank + dr);
  for (int i = threadIdx.x; i < rank; i += blockDim.x) dst[i] = from_f32<T>(to_f32(row[q_rank + i]) * inv_kv * to_f32(wkv[i]));
  const T* kr = row + q_rank + rank;
  const float pos = (float)positions[t];
  const int half = rot_dims / 2;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    const float u = to_f32(kr[i]), v = to_f32(kr[i + half]);
    dst[rank + i] = from_f32<T>(u * cs - v * sn);
    dst[rank + i + half] = from_f32<T>(v * cs + u * sn);
  }
  for (int i = rot_dims + threadIdx.x; i < dr; i += blockDim.x) dst[rank + i] = kr[i];
}

// ------------------------------------------------------------------------------------------ attention
struct LatentAttnParams {
  const void* qa;        // [tokens, H, rank] through (qa_st, qa_sh)
  const void* qr;        // unrotated rope part of q: element (t, h, i) at qr + t * qr_st + h * qr_sh + i
  void* out;             // [tokens, H, rank] through (o_st, o_sh)
  const void* cache;     // [slots, rank + dr]
  const void* gate;      // per-(token, head) gate logits, or null
  const int32_t* req_to_token;
  const int64_t* req_pool_indices;
  const int32_t* tok_req;     // null: token t belongs to sequence t
  const int64_t* positions;
  const int32_t* blocks;      // pairs (first token, count) of runs inside one sequence, or null: one token per run
  const float* sink;          // [H]
  const float* inv_freq;      // [rot_dims / 2]
  int64_t qa_st, qa_sh, qr_st, qr_sh, o_st, o_sh, gate_st, rtt_stride;
  int H, rank, dr, rot_dims, window, hg, kb, rows_cap;
  float scale;
  // matrix-core kernel only: the keys of a run cut into nsplit ranges, one workgroup each; unnormalised partial
  // sums, maxima and denominators go to part_o / part_m / part_l ([nsplit][tokens][H][...]) for the merge kernel
  int nsplit;
  int64_t tokens;
  float* part_o;
  float* part_m;
  float* part_l;
};

struct LatentAttnPlan {
  int hg;        // heads per workgroup
  int bq;        // tokens per workgroup
  int kb;        // cache rows per LDS tile
  size_t lds;
};

inline size_t latent_attn_lds(int m, int kb, int rank, int dr) {
  const int rp = (rank + dr) | 1;
  return sizeof(float) * ((size_t)m * rp + (size_t)kb * rp + (size_t)m * rank + (size_t)m * kb + 3 * (size_t)m) + sizeof(int) * kb;
}

inline LatentAttnPlan plan_latent_attn(int H, int rank, int dr) {
  LatentAttnPlan p;
  p.hg = std::min(H, 32);
  p.bq = p.hg == H ? std::max(1, 32 / p.hg) : 1;
  p.kb = 32;
  const size_t budget = 150 * 1024;
  while (latent_attn_lds(p.hg * p.bq, p.kb, rank, dr) > budget && p.kb > 8) p.kb /= 2;
  while (latent_attn_lds(p.hg * p.bq, p.kb, rank, dr) > budget && p.bq > 1) p.bq -= 1;
  while (latent_attn_lds(p.hg * p.bq, p.kb, rank, dr) > budget && p.hg > 1) p.hg = (p.hg + 1) / 2;
  p.lds = latent_attn_lds(p.hg * p.bq, p.kb, rank, dr);
  return p;
}

template <typename T>
__global__ __launch_bounds__(256) void latent_window_attention_kernel(const LatentAttnParams p) {
  extern __shared__ __attribute__((aligned(16))) float smf[];
  const int rank = p.rank, dr = p.dr, R = rank + dr, rp = R | 1, KB = p.kb;
  int t0, n;
  if (p.blocks) {
    t0 = p.blocks[2 * blockIdx.x];
    n = p.blocks[2 * blockIdx.x + 1];
  } else {
    t0 = blockIdx.x;
    n = 1;
  }
  const int h0 = blockIdx.y * p.hg;
  const int nh = min(p.hg, p.H - h0);
  const int M = n * nh;
  // LDS carve-up for the planned row count (the launch reserved bytes for rows_cap = hg * bq rows)
  const int rows_cap = p.rows_cap;
  float* Q = smf;                                // [rows_cap][rp]
  float* K = Q + (size_t)rows_cap * rp;          // [KB][rp]
  float* O = K + (size_t)KB * rp;                // [rows_cap][rank]
  float* S = O + (size_t)rows_cap * rank;        // [rows_cap][KB]
  float* mrow = S + (size_t)rows_cap * KB;
  float* lrow = mrow + rows_cap;
  float* arow = lrow + rows_cap;
  int* kslot = reinterpret_cast<int*>(arow + rows_cap);

  const T* qa = static_cast<const T*>(p.qa);
  const T* qr = static_cast<const T*>(p.qr);
  const T* cache = static_cast<const T*>(p.cache);
  const int b = p.tok_req ? p.tok_req[t0] : t0;
  const int64_t p0 = p.positions[t0];
  const int32_t* table = p.req_to_token + p.req_pool_indices[b] * p.rtt_stride;
  const int tid = threadIdx.x, nt = blockDim.x;

  // ---- queries: absorbed part as is, rope part rotated by the token's position
  for (int idx = tid; idx < M * rank; idx += nt) {
    const int m = idx / rank, r = idx - m * rank;
    const int ti = m / nh, hi = m - ti * nh;
    Q[(size_t)m * rp + r] = to_f32(qa[(int64_t)(t0 + ti) * p.qa_st + (int64_t)(h0 + hi) * p.qa_sh + r]);
  }
  const int half = p.rot_dims / 2;
  for (int idx = tid; idx < M * half; idx += nt) {
    const int m = idx / half, i = idx - m * half;
    const int ti = m / nh, hi = m - ti * nh;
    const T* src = qr + (int64_t)(t0 + ti) * p.qr_st + (int64_t)(h0 + hi) * p.qr_sh;
    float sn, cs;
    sincosf((float)(p0 + ti) * p.inv_freq[i], &sn, &cs);
    const float u = to_f32(src[i]), v = to_f32(src[i + half]);
    Q[(size_t)m * rp + rank + i] = u * cs - v * sn;
    Q[(size_t)m * rp + rank + i + half] = v * cs + u * sn;
  }
  const int tail = dr - p.rot_dims;
  for (int idx = tid; idx < M * tail; idx += nt) {
    const int m = idx / tail, i = p.rot_dims + (idx - m * tail);
    const int ti = m / nh, hi = m - ti * nh;
    Q[(size_t)m * rp + rank + i] = to_f32(qr[(int64_t)(t0 + ti) * p.qr_st + (int64_t)(h0 + hi) * p.qr_sh + i]);
  }
  for (int idx = tid; idx < M * rank; idx += nt) O[idx] = 0.f;
  for (int m = tid; m < M; m += nt) {
    mrow[m] = p.sink[h0 + (m % nh)];
    lrow[m] = 1.0f;
  }
  __syncthreads();

  const int64_t j_hi = p0 + n - 1;
  const int64_t j_lo = max((int64_t)0, p0 - (int64_t)p.window + 1);
  for (int64_t j0 = j_lo; j0 <= j_hi; j0 += KB) {
    const int kn = (int)min((int64_t)KB, j_hi - j0 + 1);
    for (int jj = tid; jj < kn; jj += nt) kslot[jj] = table[j0 + jj];
    __syncthreads();
    for (int idx = tid; idx < kn * R; idx += nt) {
      const int jj = idx / R, r = idx - jj * R;
      K[(size_t)jj * rp + r] = to_f32(cache[(int64_t)kslot[jj] * R + r]);
    }
    __syncthreads();
    // ---- scores
    for (int idx = tid; idx < M * KB; idx += nt) {
      const int m = idx / KB, jj = idx - m * KB;
      float s = -INFINITY;
      if (jj < kn) {
        const int64_t j = j0 + jj, pq = p0 + m / nh;
        if (j <= pq && pq - j < p.window) {
          const float* qrow = Q + (size_t)m * rp;
          const float* krow = K + (size_t)jj * rp;
          float acc = 0.f;
          for (int r = 0; r < R; ++r) acc = fmaf(qrow[r], krow[r], acc);
          s = acc * p.scale;
        }
      }
      S[(size_t)m * KB + jj] = s;
    }
    __syncthreads();
    // ---- running softmax per row
    for (int m = tid; m < M; m += nt) {
      float* srow = S + (size_t)m * KB;
      const float mo = mrow[m];
      float mx = mo;
      for (int jj = 0; jj < kn; ++jj) mx = fmaxf(mx, srow[jj]);
      const float alpha = expf(mo - mx);
      float sum = 0.f;
      for (int jj = 0; jj < kn; ++jj) {
        const float e = expf(srow[jj] - mx);   // exp(-inf) = 0 for masked keys
        srow[jj] = e;
        sum += e;
      }
      mrow[m] = mx;
      lrow[m] = lrow[m] * alpha + sum;
      arow[m] = alpha;
    }
    __syncthreads();
    // ---- weighted sum of the latent rows
    for (int idx = tid; idx < M * rank; idx += nt) {
      const int m = idx / rank, r = idx - m * rank;
      const float* srow = S + (size_t)m * KB;
      float acc = O[idx] * arow[m];
      for (int jj = 0; jj < kn; ++jj) acc = fmaf(srow[jj], K[(size_t)jj * rp + r], acc);
      O[idx] = acc;
    }
    __syncthreads();
  }
  T* out = static_cast<T*>(p.out);
  const T* gate = static_cast<const T*>(p.gate);
  for (int idx = tid; idx < M * rank; idx += nt) {
    const int m = idx / rank, r = idx - m * rank;
    const int ti = m / nh, hi = m - ti * nh;
    float o = O[idx] / lrow[m];
    if (gate) o *= 1.0f / (1.0f + expf(-to_f32(gate[(int64_t)(t0 + ti) * p.gate_st + h0 + hi])));
    out[(int64_t)(t0 + ti) * p.o_st + (int64_t)(h0 + hi) * p.o_sh + r] = from_f32<T>(o);
  }
}


// ------------------------------------------------------------------------------------------ matrix-core kernel (16-bit)
// 64 query rows (tokens x heads) per workgroup, 16 per wave; cache rows in LDS tiles of 32 keys shared by the four
// waves.  S = Q K^T on v_mfma_f32_16x16x32 (both operands read as 16-byte fragments of their LDS rows, so the number
// of 32-wide chunks is a run-time loop), softmax on the fp32 accumulators (a row's 32 scores sit in 16 lanes x 2
// registers), P rounded to T and passed through LDS into the A layout of v_mfma_f32_16x16x16, whose B operand -- the
// value part of the same K tile -- comes from a transposed LDS read.  NRT = 16-column tiles of the value part kept
// in registers (compile time: 4 accumulators each).
// Reductions over the 16 lanes that hold one row's scores, on the data-parallel-primitive path of the vector ALU
// (quad swaps, then the mirror of each half row, then the mirror of the row) instead of LDS permutes.
template <int CTRL> __device__ __forceinline__ float lm_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float lm_row16_max(float v) {
  v = fmaxf(v, lm_dpp<0xB1>(v));
  v = fmaxf(v, lm_dpp<0x4E>(v));
  v = fmaxf(v, lm_dpp<0x141>(v));
  return fmaxf(v, lm_dpp<0x140>(v));
}
__device__ __forceinline__ float lm_row16_sum(float v) {
  v += lm_dpp<0xB1>(v);
  v += lm_dpp<0x4E>(v);
  v += lm_dpp<0x141>(v);
  return v + lm_dpp<0x140>(v);
}

constexpr int LM_KB = 32;
constexpr int LM_ROWS = 64;
// rows a prefill workgroup aims for: 32 (two computing waves) so that two workgroups share a CU and one's K-tile
// loads overlap the other's products; head counts above 32 take one token of up to 64 heads
constexpr int LM_PREFILL_ROWS = 32;
inline int lm_block_tokens(int heads) { return heads >= LM_PREFILL_ROWS ? 1 : LM_PREFILL_ROWS / heads; }
constexpr int LM_PLD = LM_KB + 8;

inline int lm_ld(int rank, int dr) { return ((rank + dr + 31) & ~31) + 8; }
inline size_t lm_lds_bytes(int rank, int dr, int rows = LM_ROWS) {
  return 2 * ((size_t)rows * lm_ld(rank, dr) + (size_t)LM_KB * lm_ld(rank, dr) + (size_t)rows * LM_PLD) + sizeof(float) * 2 * rows;
}

// ROWS: query rows the workgroup holds: 16, 32 or 64 (the smallest that takes the run's tokens x heads); with 16 or 32
// two workgroups share a CU
template <typename T, int NRT, int ROWS>
__global__ __launch_bounds__(256) void latent_window_attention_mfma_kernel(const LatentAttnParams p) {
  extern __shared__ __attribute__((aligned(16))) char sm_raw[];
  using frag = typename Mfma<T>::frag;
  using frag4 = typename Mfma16<T>::frag;
  const int rank = p.rank, dr = p.dr, R = rank + dr;
  const int RP = (R + 31) & ~31, LD = RP + 8;
  T* Qs = reinterpret_cast<T*>(sm_raw);                 // [64][LD]
  T* Ks = Qs + (size_t)ROWS * LD;                       // [32][LD]
  T* Ps = Ks + (size_t)LM_KB * LD;                      // [ROWS][LM_PLD]: the tile's softmax weights, rounded to T
  float* alpha_s = reinterpret_cast<float*>(Ps + (size_t)ROWS * LM_PLD);   // [ROWS]: this tile's rescale of the running sums
  float* l_s = alpha_s + ROWS;                                              // [ROWS]: final denominators
  int t0, n;
  if (p.blocks) {
    t0 = p.blocks[2 * blockIdx.x];
    n = p.blocks[2 * blockIdx.x + 1];
  } else {
    t0 = blockIdx.x;
    n = 1;
  }
  const int h0 = blockIdx.y * p.hg;
  const int nh = min(p.hg, p.H - h0);
  const int M = n * nh;
  const int split = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, lg = lane >> 4;
  const T* qa = static_cast<const T*>(p.qa);
  const T* qr = static_cast<const T*>(p.qr);
  const T* cache = static_cast<const T*>(p.cache);
  const int b = p.tok_req ? p.tok_req[t0] : t0;
  const int64_t p0 = p.positions[t0];
  const int32_t* table = p.req_to_token + p.req_pool_indices[b] * p.rtt_stride;

  // ---- the keys of this workgroup
  int64_t j_hi = p0 + n - 1;
  int64_t j_lo = max((int64_t)0, p0 - (int64_t)p.window + 1);
  if (p.nsplit > 1) {
    const int64_t keys = j_hi - j_lo + 1;
    const int64_t chunk = ((keys + p.nsplit - 1) / p.nsplit + LM_KB - 1) / LM_KB * LM_KB;
    j_lo += split * chunk;
    j_hi = min(j_hi, j_lo + chunk - 1);
  }

  // ---- queries into LDS: absorbed part as is, rope part rotated in fp32 and rounded, padding zero.  A wave takes
  // whole rows (no per-element division); the absorbed part moves as 16-byte vectors when the strides allow it.
  {
    const bool qvec = (rank % 8 == 0) && (p.qa_st % 8 == 0) && (p.qa_sh % 8 == 0) && aligned16(qa);
    const int half = p.rot_dims >> 1;
    for (int m = wave; m < ROWS; m += 4) {
      T* dst = Qs + (size_t)m * LD;
      if (m >= M) {
        for (int r = 8 * lane; r < RP; r += 512) stvec<T, 8>(dst + r, Vec<T, 8>{});
        continue;
      }
      const int ti = m / nh, hi = m - ti * nh;
      const T* src = qa + (int64_t)(t0 + ti) * p.qa_st + (int64_t)(h0 + hi) * p.qa_sh;
      if (qvec) {
        for (int r = 8 * lane; r < rank; r += 512) stvec<T, 8>(dst + r, ldvec<T, 8>(src + r));
      } else {
        for (int r = lane; r < rank; r += 64) dst[r] = src[r];
      }
      const T* rs = qr + (int64_t)(t0 + ti) * p.qr_st + (int64_t)(h0 + hi) * p.qr_sh;
      const float pos = (float)(p0 + ti);
      for (int i = lane; i < half; i += 64) {
        float sn, cs;
        sincosf(pos * p.inv_freq[i], &sn, &cs);
        const float u = to_f32(rs[i]), w = to_f32(rs[i + half]);
        dst[rank + i] = from_f32<T>(u * cs - w * sn);
        dst[rank + i + half] = from_f32<T>(w * cs + u * sn);
      }
      for (int i = p.rot_dims + lane; i < dr; i += 64) dst[rank + i] = rs[i];
      for (int r = R + lane; r < RP; r += 64) dst[r] = from_f32<T>(0.f);
    }
  }

  // ---- running softmax state of this lane's four rows (rows 16 wave + 4 lg + r), replicated over the 16 lanes
  // Scores and softmax go by ROWS: wave w owns the 16 rows of row tile w.  The products with V go by COLUMNS: wave w
  // owns column tiles w CT .. w CT + CT - 1 of the result for every row tile, so that each V fragment is read from LDS
  // once per workgroup and serves all row tiles; the weights P and the rescale factors cross between the waves in LDS.
  constexpr int RT = ROWS / 16, CT = NRT / 4;
  const int r0 = 16 * wave;
  const bool wave_has_rows = r0 < ROWS;
  float mrun[4], lrun[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int m = r0 + 4 * lg + r;
    const bool with_sink = split == 0 && m < M;
    mrun[r] = with_sink ? p.sink[h0 + (m % nh)] * 1.4426950408889634f : -1e30f;     // base-2 units, as the scores
    lrun[r] = with_sink ? 1.0f : 0.0f;
  }
  f32x4 acc[RT][CT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int c = 0; c < CT; ++c) acc[rt][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bool vec_ok = (R % 8 == 0) && aligned16(cache);
  __syncthreads();

  for (int64_t j0 = j_lo; j0 <= j_hi; j0 += LM_KB) {
    const int kn = (int)min((int64_t)LM_KB, j_hi - j0 + 1);
    // wave w brings rows w, w + 4, ..: four rows per round, each lane up to two 16-byte pieces of a row, all of a
    // round's loads issued before the first store; rows past the last key and columns past R are zero
#pragma unroll
    for (int rb = 0; rb < LM_KB / 4; rb += 4) {
      Vec<T, 8> v[4][2];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int jj = wave + 4 * (rb + q);
        const T* row = cache + (int64_t)(jj < kn ? table[j0 + jj] : 0) * R;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int r = 8 * (lane + 64 * e);
          Vec<T, 8> x{};
          if (jj < kn && r < R) {
            if (vec_ok && r + 8 <= R) {
              x = ldvec<T, 8>(row + r);
            } else {
#pragma unroll
              for (int k = 0; k < 8; ++k)
                if (r + k < R) x.v[k] = row[r + k];
            }
          }
          v[q][e] = x;
        }
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int jj = wave + 4 * (rb + q);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int r = 8 * (lane + 64 * e);
          if (r < RP) stvec<T, 8>(Ks + (size_t)jj * LD + r, v[q][e]);
        }
      }
    }
    __syncthreads();
    if (wave_has_rows) {
      // ---- scores of 16 rows x 32 keys
      f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
      const T* qrow = Qs + (size_t)(r0 + li) * LD + 8 * lg;
      const T* k0row = Ks + (size_t)li * LD + 8 * lg;
      const T* k1row = Ks + (size_t)(16 + li) * LD + 8 * lg;
      // three 32-wide chunks per round: nine LDS reads in flight before the six products that use them
      int kc = 0;
      for (; kc + 96 <= RP; kc += 96) {
        frag a[3], b0[3], b1[3];
#pragma unroll
        for (int u = 0; u < 3; ++u) {
          a[u] = *reinterpret_cast<const frag*>(qrow + kc + 32 * u);
          b0[u] = *reinterpret_cast<const frag*>(k0row + kc + 32 * u);
          b1[u] = *reinterpret_cast<const frag*>(k1row + kc + 32 * u);
        }
#pragma unroll
        for (int u = 0; u < 3; ++u) {
          s0 = Mfma<T>::run(a[u], b0[u], s0);
          s1 = Mfma<T>::run(a[u], b1[u], s1);
        }
      }
      for (; kc < RP; kc += 32) {
        const frag a = *reinterpret_cast<const frag*>(qrow + kc);
        s0 = Mfma<T>::run(a, *reinterpret_cast<const frag*>(k0row + kc), s0);
        s1 = Mfma<T>::run(a, *reinterpret_cast<const frag*>(k1row + kc), s1);
      }
      // softmax in base 2: exp(x) = 2^(x log2 e), with the scale folded into the factor; the four rows' reductions are
      // independent chains
      float pr[2][4], alpha[4], sv[2][4], mx[4];
      const float sl2 = p.scale * 1.4426950408889634f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = r0 + 4 * lg + r;
        const int64_t pq = p0 + m / nh;
        const float raw[2] = {s0[r], s1[r]};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int64_t j = j0 + 16 * h + li;
          const bool vis = m < M && j <= j_hi && j <= pq && pq - j < p.window;
          sv[h][r] = vis ? raw[h] * sl2 : -INFINITY;
        }
        mx[r] = fmaxf(sv[0][r], sv[1][r]);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) mx[r] = lm_row16_max(mx[r]);
      float sum[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float mnew = fmaxf(mrun[r], mx[r]);
        alpha[r] = exp2f(mrun[r] - mnew);
        pr[0][r] = exp2f(sv[0][r] - mnew);
        pr[1][r] = exp2f(sv[1][r] - mnew);
        sum[r] = pr[0][r] + pr[1][r];
        mrun[r] = mnew;
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) lrun[r] = lrun[r] * alpha[r] + lm_row16_sum(sum[r]);
      T* pw = Ps + (size_t)r0 * LM_PLD;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pw[(4 * lg + r) * LM_PLD + li] = from_f32<T>(pr[0][r]);
        pw[(4 * lg + r) * LM_PLD + 16 + li] = from_f32<T>(pr[1][r]);
        if (li == 0) alpha_s[r0 + 4 * lg + r] = alpha[r];
      }
    }
    __syncthreads();
    // ---- O += P V on the k = 32 instruction: lane group lg supplies keys 8 lg .. 8 lg + 7 of the tile, as two
    // transposed reads of four keys each; V = the first `rank` columns of the K tile.  This wave's CT column tiles:
    // all their reads first, then every row tile's products.
    {
      const T* vrow = Ks + (size_t)(8 * lg + (li >> 2)) * LD + 4 * (li & 3) + 16 * CT * wave;
      typename TrRead<T>::v4 lo[CT], hi[CT];
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        if (16 * (CT * wave + c) < rank) {
          lo[c] = TrRead<T>::run(vrow + 16 * c);
          hi[c] = TrRead<T>::run(vrow + 4 * LD + 16 * c);
        }
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const frag pa = *reinterpret_cast<const frag*>(Ps + (size_t)(16 * rt + li) * LM_PLD + 8 * lg);
        const f32x4 al = *reinterpret_cast<const f32x4*>(alpha_s + 16 * rt + 4 * lg);
#pragma unroll
        for (int c = 0; c < CT; ++c) {
          if (16 * (CT * wave + c) < rank) {
            typename TrRead<T>::v4 both[2] = {lo[c], hi[c]};
            f32x4 o = acc[rt][c];
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] *= al[r];
            acc[rt][c] = Mfma<T>::run(pa, __builtin_bit_cast(frag, both), o);
          }
        }
      }
    }
    __syncthreads();
  }
  // ---- epilogue: the row owners publish the denominators (and, for a key range, the range's maximum and sum); then
  // every wave writes its columns of all rows: this lane holds rows 16 rt + 4 lg + r, columns 16 (CT wave + c) + li
  if (wave_has_rows) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = r0 + 4 * lg + r;
      if (li == 0) l_s[m] = lrun[r];
      if (p.nsplit > 1 && li == 0 && m < M) {
        const int ti = m / nh, hi = m - ti * nh;
        const int64_t cell = ((int64_t)split * p.tokens + (t0 + ti)) * p.H + (h0 + hi);
        p.part_m[cell] = mrun[r];
        p.part_l[cell] = lrun[r];
      }
    }
  }
  __syncthreads();
  T* out = static_cast<T*>(p.out);
  const T* gate = static_cast<const T*>(p.gate);
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = 16 * rt + 4 * lg + r;
      if (m >= M) continue;
      const int ti = m / nh, hi = m - ti * nh;
      const int64_t t = t0 + ti;
      const int h = h0 + hi;
      if (p.nsplit > 1) {
        const int64_t cell = ((int64_t)split * p.tokens + t) * p.H + h;
#pragma unroll
        for (int c = 0; c < CT; ++c) {
          const int col = 16 * (CT * wave + c) + li;
          if (col < rank) p.part_o[cell * rank + col] = acc[rt][c][r];
        }
      } else {
        float f = 1.0f / l_s[m];
        if (gate) f *= 1.0f / (1.0f + expf(-to_f32(gate[t * p.gate_st + h])));
#pragma unroll
        for (int c = 0; c < CT; ++c) {
          const int col = 16 * (CT * wave + c) + li;
          if (col < rank) out[t * p.o_st + (int64_t)h * p.o_sh + col] = from_f32<T>(acc[rt][c][r] * f);
        }
      }
    }
  }
}

// One workgroup per (token, head): out = sum_i o_i exp(m_i - m) / sum_i l_i exp(m_i - m), times the gate.  The split
// weights are computed once into LDS; every thread then sums four columns at a time.
template <typename T>
__global__ __launch_bounds__(128) void latent_window_merge_kernel(const LatentAttnParams p) {
  __shared__ float wz[64];
  __shared__ float fsh;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int ns = p.nsplit;
  if (threadIdx.x < 64) {
    const int z = threadIdx.x;
    const int64_t cell = ((int64_t)z * p.tokens + t) * p.H + h;
    const float m = z < ns ? p.part_m[cell] : -1e30f;
    const float mx = wave_max(m);
    const float w = z < ns ? exp2f(m - mx) : 0.f;
    const float den = wave_sum(z < ns ? p.part_l[cell] * w : 0.f);
    wz[z] = w;
    if (z == 0) {
      float f = 1.0f / den;
      const T* gate = static_cast<const T*>(p.gate);
      if (gate) f *= 1.0f / (1.0f + expf(-to_f32(gate[t * p.gate_st + h])));
      fsh = f;
    }
  }
  __syncthreads();
  const float f = fsh;
  T* out = static_cast<T*>(p.out) + t * p.o_st + (int64_t)h * p.o_sh;
  const int64_t cell0 = (t * p.H + h) * (int64_t)p.rank, zstride = p.tokens * p.H * (int64_t)p.rank;
  if (p.rank % 4 == 0) {
    for (int c = 4 * threadIdx.x; c < p.rank; c += 4 * 128) {
      float4 o = float4{0.f, 0.f, 0.f, 0.f};
      for (int z = 0; z < ns; ++z) {
        const float4 v = *reinterpret_cast<const float4*>(p.part_o + z * zstride + cell0 + c);
        const float w = wz[z];
        o.x += v.x * w; o.y += v.y * w; o.z += v.z * w; o.w += v.w * w;
      }
      out[c] = from_f32<T>(o.x * f); out[c + 1] = from_f32<T>(o.y * f);
      out[c + 2] = from_f32<T>(o.z * f); out[c + 3] = from_f32<T>(o.w * f);
    }
  } else {
    for (int c = threadIdx.x; c < p.rank; c += 128) {
      float o = 0.f;
      for (int z = 0; z < ns; ++z) o += p.part_o[z * zstride + cell0 + c] * wz[z];
      out[c] = from_f32<T>(o * f);
    }
  }
}

template <typename T> inline bool launch_latent_mfma(const LatentAttnParams& p, dim3 grid, int rows, hipStream_t st) {
#define MI355_LM_LAUNCH(N, ROWS_)                                                                                \
  {                                                                                                              \
    auto kern = latent_window_attention_mfma_kernel<T, N, ROWS_>;                                                \
    const size_t lds = lm_lds_bytes(p.rank, p.dr, ROWS_);                                                        \
    if (lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, p);                                                       \
  }
#define MI355_LM_CASE(N)                       \
  {                                            \
    if (rows <= 16) MI355_LM_LAUNCH(N, 16)     \
    else if (rows <= 32) MI355_LM_LAUNCH(N, 32) \
    else MI355_LM_LAUNCH(N, LM_ROWS)           \
  }
  const int tiles = (p.rank + 15) / 16;
  if (tiles <= 4) MI355_LM_CASE(4)
  else if (tiles <= 8) MI355_LM_CASE(8)
  else if (tiles <= 16) MI355_LM_CASE(16)
  else if (tiles <= 32) MI355_LM_CASE(32)
  else return false;
#undef MI355_LM_CASE
#undef MI355_LM_LAUNCH
  return true;
}

inline bool latent_mfma_serves(int dtype, int rank, int dr) {
  // (a row of the K tile is at most 2 x 64 pieces of 16 bytes: the loader's two pieces per lane)
  return (dtype == MI355_BF16 || dtype == MI355_F16) && rank <= 512 && rank + dr <= 1024 && lm_lds_bytes(rank, dr) <= 160 * 1024;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

int mi355_latent_norms_rope_write(void* cq, void* cache, const void* a, const void* q_weight, const void* kv_weight,
                                  const int64_t* positions, const int64_t* out_cache_loc, const float* inv_freq, int64_t tokens,
                                  int64_t a_stride, int q_rank, int rank, int rope_dim, int rot_dims, int64_t num_slots, float eps,
                                  int dtype, void* stream) {
  MI355_REQUIRE(cq && cache && a && q_weight && kv_weight && positions && out_cache_loc && inv_freq, MI355_ERR_INVALID,
                "latent_norms_rope_write: null pointer");
  MI355_REQUIRE(tokens >= 0 && q_rank > 0 && rank > 0 && rope_dim >= 0 && rot_dims >= 0 && rot_dims <= rope_dim && rot_dims % 2 == 0 &&
                    a_stride >= (int64_t)q_rank + rank + rope_dim && num_slots > 0,
                MI355_ERR_INVALID, "latent_norms_rope_write: bad shape");
  if (tokens == 0) return MI355_OK;
  MI355_DISPATCH_DTYPE(dtype, "latent_norms_rope_write", {
    hipLaunchKernelGGL((latent_norms_rope_write_kernel<T>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, (T*)cq,
                       (T*)cache, (const T*)a, (const T*)q_weight, (const T*)kv_weight, positions, out_cache_loc, inv_freq, a_stride,
                       q_rank, rank, rope_dim, rot_dims, eps);
  });
  MI355_CHECK_LAUNCH("latent_norms_rope_write");
  return MI355_OK;
}

int mi355_latent_window_attention_block_tokens(int heads, int rank, int rope_dim, int dtype) {
  if (heads <= 0 || rank <= 0 || rope_dim < 0) return 0;
  if (latent_mfma_serves(dtype, rank, rope_dim)) return lm_block_tokens(heads);
  const LatentAttnPlan pl = plan_latent_attn(heads, rank, rope_dim);
  return pl.lds <= 160 * 1024 ? pl.bq : 0;
}

int mi355_latent_window_attention(void* out, const void* qa, const void* qr, const void* cache, const void* gate,
                                  const int32_t* req_to_token, const int64_t* req_pool_indices, const int32_t* tok_req,
                                  const int64_t* positions, const int32_t* blocks, int64_t num_blocks, const float* sink,
                                  const float* inv_freq, int64_t qa_token_stride, int64_t qa_head_stride, int64_t qr_token_stride,
                                  int64_t qr_head_stride, int64_t out_token_stride, int64_t out_head_stride, int64_t gate_stride,
                                  int64_t req_to_token_stride, int heads, int rank, int rope_dim, int rot_dims, int window,
                                  float scale, int num_splits, float* split_scratch, int64_t tokens, int dtype, void* stream) {
  MI355_REQUIRE(out && qa && cache && req_to_token && req_pool_indices && positions && sink, MI355_ERR_INVALID,
                "latent_window_attention: null pointer");
  MI355_REQUIRE(rope_dim == 0 || (qr && inv_freq), MI355_ERR_INVALID, "latent_window_attention: the rope part needs qr and inv_freq");
  MI355_REQUIRE(heads > 0 && rank > 0 && rope_dim >= 0 && rot_dims >= 0 && rot_dims <= rope_dim && rot_dims % 2 == 0 && window > 0 &&
                    num_blocks >= 0 && num_blocks < (1ll << 31),
                MI355_ERR_INVALID, "latent_window_attention: bad shape");
  if (num_blocks == 0) return MI355_OK;
  const bool mfma = latent_mfma_serves(dtype, rank, rope_dim);
  MI355_REQUIRE(num_splits >= 1 && num_splits <= 64 && (num_splits == 1 || (mfma && blocks == nullptr && split_scratch && tokens == num_blocks)),
                MI355_ERR_INVALID, "latent_window_attention: key splits need the 16-bit kernel, one token per run and a scratch array");
  LatentAttnPlan pl = plan_latent_attn(heads, rank, rope_dim);
  if (mfma) {
    pl.hg = std::min(heads, LM_ROWS);
    pl.bq = lm_block_tokens(heads);
    pl.kb = LM_KB;
    pl.lds = lm_lds_bytes(rank, rope_dim);
  }
  MI355_REQUIRE(pl.lds <= 160 * 1024, MI355_ERR_UNSUPPORTED, "latent_window_attention: rank %d + rope %d does not fit the LDS tile", rank,
                rope_dim);
  LatentAttnParams p;
  p.qa = qa; p.qr = qr; p.out = out; p.cache = cache; p.gate = gate;
  p.req_to_token = req_to_token; p.req_pool_indices = req_pool_indices; p.tok_req = tok_req; p.positions = positions;
  p.blocks = blocks; p.sink = sink; p.inv_freq = inv_freq;
  p.qa_st = qa_token_stride; p.qa_sh = qa_head_stride; p.qr_st = qr_token_stride; p.qr_sh = qr_head_stride;
  p.o_st = out_token_stride; p.o_sh = out_head_stride; p.gate_st = gate_stride; p.rtt_stride = req_to_token_stride;
  p.H = heads; p.rank = rank; p.dr = rope_dim; p.rot_dims = rot_dims; p.window = window; p.hg = pl.hg; p.kb = pl.kb; p.rows_cap = pl.hg * pl.bq;
  p.scale = scale;
  p.nsplit = num_splits; p.tokens = tokens;
  p.part_o = split_scratch;
  p.part_m = split_scratch ? split_scratch + (int64_t)num_splits * tokens * heads * rank : nullptr;
  p.part_l = split_scratch ? p.part_m + (int64_t)num_splits * tokens * heads : nullptr;
  if (mfma) {
    const dim3 mgrid((unsigned)num_blocks, (unsigned)((heads + pl.hg - 1) / pl.hg), (unsigned)num_splits);
    bool ok = false;
    const int rows = blocks == nullptr ? pl.hg : pl.hg * pl.bq;     // one token per run: a workgroup holds at most hg rows
    if (dtype == MI355_BF16) ok = launch_latent_mfma<bf16_t>(p, mgrid, rows, (hipStream_t)stream);
    else ok = launch_latent_mfma<f16_t>(p, mgrid, rows, (hipStream_t)stream);
    MI355_REQUIRE(ok, MI355_ERR_UNSUPPORTED, "latent_window_attention: rank %d is not served", rank);
    MI355_CHECK_LAUNCH("latent_window_attention");
    if (num_splits > 1) {
      const dim3 g2((unsigned)tokens, (unsigned)heads);
      if (dtype == MI355_BF16) hipLaunchKernelGGL((latent_window_merge_kernel<bf16_t>), g2, dim3(128), 0, (hipStream_t)stream, p);
      else hipLaunchKernelGGL((latent_window_merge_kernel<f16_t>), g2, dim3(128), 0, (hipStream_t)stream, p);
      MI355_CHECK_LAUNCH("latent_window_attention (merge)");
    }
    return MI355_OK;
  }
  const dim3 grid((unsigned)num_blocks, (unsigned)((heads + pl.hg - 1) / pl.hg), 1);
  MI355_DISPATCH_DTYPE(dtype, "latent_window_attention", {
    auto kern = latent_window_attention_kernel<T>;
    if (pl.lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds);
    hipLaunchKernelGGL(kern, grid, dim3(256), pl.lds, (hipStream_t)stream, p);
  });
  MI355_CHECK_LAUNCH("latent_window_attention");
  return MI355_OK;
}
