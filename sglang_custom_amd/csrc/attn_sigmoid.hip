// Causal attention whose weights are NOT normalised over the keys:
//     out[t, h] = sum_{j <= pos(t)} sigmoid((q[t, h] . K[j, g]) * scale * temp[h] + bias[h]) * V[j, g],   g = h / (H / G)
// over per-layer key / value buffers [slots, G, d] / [slots, G, dv] reached through the request table.  Scores and weights
// are fp32.  Because nothing is normalised, a token's keys can be cut into ranges whose partial sums simply add: a decode
// step with few sequences does that (num_splits > 1, partial sums in fp32 scratch, a second launch adds them in a fixed
// order).
//
// A workgroup takes one run of consecutive tokens of one sequence, one kv head and up to SG_ROWS (token, query head) rows
// of it: the heads of the group that share the kv head ride along with the tokens, so a decode step still fills the row
// tile with the group's heads.  K and V tiles of SG_KT keys are staged in LDS once per workgroup.
//   * 16-bit dtypes, d and dv multiples of 32: matrix cores (16x16x32 MFMA for Q K^T from LDS rows, the weights through
//     LDS in the activation dtype, 16x16x16 MFMA for P V with V read by columns),
//   * everything else (fp32, odd widths): vector ALU with the same tiling, all fp32.
#include "common.cuh"

#include <algorithm>
#include <type_traits>

namespace mi355 {
namespace {

constexpr int SG_ROWS = 16;
constexpr int SG_KT = 32;

__device__ __forceinline__ float sg_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
// The same on the hardware's exp2 and reciprocal (about one ulp each): for weights that are rounded to a 16-bit type right
// after.  exp(-z) = inf gives 0, as it should.
__device__ __forceinline__ float sg_sigmoid_fast(float z) { return __frcp_rn(1.0f + __expf(-z)); }

struct SgArgs {
  void* out;
  float* partial;
  const void* q;
  const void* k_cache;
  const void* v_cache;
  const int32_t* req_to_token;
  const int64_t* req_pool_indices;
  const int32_t* tok_req;
  const int64_t* positions;
  const int32_t* blocks;
  const float* temp;
  const float* bias;
  int64_t q_token_stride, q_head_stride, out_token_stride, out_head_stride, req_to_token_stride, tokens;
  int heads, kv_heads, d, dv, heads_per_tile, tokens_per_tile, num_splits;
  float scale;
};

// Vector-ALU kernel.  sm: Qs [16][d] | Ks [KT][d + 1] | Vs [KT][dv] | Ps [16][KT]
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_attention_valu_kernel(SgArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int d = a.d, dv = a.dv;
  float* Qs = sm;
  float* Ks = Qs + SG_ROWS * d;
  float* Vs = Ks + SG_KT * (d + 1);
  float* Ps = Vs + SG_KT * dv;
  __shared__ int row_pos[SG_ROWS];
  const int rep = a.heads / a.kv_heads;
  const int chunks = (rep + a.heads_per_tile - 1) / a.heads_per_tile;
  const int g = blockIdx.y / chunks, hc = blockIdx.y - g * chunks;
  const int split = blockIdx.z;
  // runs come in token order, so a sequence's later (longer) runs are listed last: take them first
  const unsigned bx = gridDim.x - 1 - blockIdx.x;
  const int64_t t0 = a.blocks != nullptr ? a.blocks[2 * bx] : bx;
  const int nt = a.blocks != nullptr ? a.blocks[2 * bx + 1] : 1;
  const int b = a.tok_req != nullptr ? a.tok_req[t0] : (int)t0;
  const int32_t* table = a.req_to_token + a.req_pool_indices[b] * a.req_to_token_stride;
  const int h0 = g * rep + hc * a.heads_per_tile;
  const int nh = min(a.heads_per_tile, rep - hc * a.heads_per_tile);
  const int tid = threadIdx.x;
  const T* q = (const T*)a.q;
  // rows: r = token * heads_per_tile + head
  for (int e = tid; e < SG_ROWS * d; e += 256) {
    const int r = e / d, i = e - r * d;
    const int tl = r / a.heads_per_tile, hl = r - tl * a.heads_per_tile;
    Qs[e] = (tl < nt && hl < nh) ? to_f32(q[(t0 + tl) * a.q_token_stride + (int64_t)(h0 + hl) * a.q_head_stride + i]) : 0.f;
  }
  if (tid < SG_ROWS) {
    const int tl = tid / a.heads_per_tile, hl = tid - tl * a.heads_per_tile;
    row_pos[tid] = (tl < nt && hl < nh) ? (int)a.positions[t0 + tl] : -1;
  }
  const int last = (int)a.positions[t0 + nt - 1];        // the run's tokens are consecutive: its last one sees the most
  const int tiles = last / SG_KT + 1;
  const int per = (tiles + a.num_splits - 1) / a.num_splits;
  const int tile_lo = split * per, tile_hi = min(tiles, tile_lo + per);
  const int r = tid >> 4, cx = tid & 15;
  const int hl_r = r % a.heads_per_tile;
  const float mul = a.scale * a.temp[h0 + min(hl_r, nh - 1)], add = a.bias[h0 + min(hl_r, nh - 1)];
  float acc[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) acc[m] = 0.f;
  const T* kc = (const T*)a.k_cache;
  const T* vc = (const T*)a.v_cache;
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const int j0 = tile * SG_KT;
    __syncthreads();
    for (int e = tid; e < SG_KT * d; e += 256) {
      const int kk = e / d, i = e - kk * d;
      const int j = j0 + kk;
      Ks[kk * (d + 1) + i] = j <= last ? to_f32(kc[((int64_t)table[j] * a.kv_heads + g) * d + i]) : 0.f;
    }
    for (int e = tid; e < SG_KT * dv; e += 256) {
      const int kk = e / dv, i = e - kk * dv;
      const int j = j0 + kk;
      Vs[e] = j <= last ? to_f32(vc[((int64_t)table[j] * a.kv_heads + g) * dv + i]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < SG_KT / 16; ++u) {
      const int kk = cx + 16 * u;
      float s = 0.f;
      for (int i = 0; i < d; ++i) s = fmaf(Qs[r * d + i], Ks[kk * (d + 1) + i], s);
      Ps[r * SG_KT + kk] = (j0 + kk <= row_pos[r]) ? sg_sigmoid(s * mul + add) : 0.f;
    }
    __syncthreads();
    for (int kk = 0; kk < SG_KT; ++kk) {
      const float p = Ps[r * SG_KT + kk];
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        const int c = cx + 16 * m;
        if (c < dv) acc[m] = fmaf(p, Vs[kk * dv + c], acc[m]);
      }
    }
  }
  const int tl = r / a.heads_per_tile, hl = r - tl * a.heads_per_tile;
  if (tl < nt && hl < nh) {
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int c = cx + 16 * m;
      if (c >= dv) continue;
      if (a.num_splits > 1) {
        a.partial[(((int64_t)split * a.tokens + t0 + tl) * a.heads + h0 + hl) * dv + c] = acc[m];
      } else {
        ((T*)a.out)[(t0 + tl) * a.out_token_stride + (int64_t)(h0 + hl) * a.out_head_stride + c] = from_f32<T>(acc[m]);
      }
    }
  }
}

// out[t, h, c] = sum over splits, in order
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_attention_sum_kernel(T* __restrict__ out, const float* __restrict__ partial,
                                                                    int64_t tokens, int heads, int dv, int num_splits,
                                                                    int64_t out_token_stride, int64_t out_head_stride) {
  const int64_t n = tokens * heads * dv;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    float s = 0.f;
    for (int k = 0; k < num_splits; ++k) s += partial[(int64_t)k * n + idx];
    const int64_t t = idx / ((int64_t)heads * dv);
    const int64_t rem = idx - t * heads * dv;
    const int h = (int)(rem / dv), c = (int)(rem - (int64_t)h * dv);
    out[t * out_token_stride + (int64_t)h * out_head_stride + c] = from_f32<T>(s);
  }
}

// Matrix-core kernel for 16-bit dtypes, d % 32 == 0, dv % 16 == 0.  Four waves, SGM_ROWS = 64 (token, head) rows.  Per key
// tile of 32:
//   S: wave w computes its 16 rows x 32 keys with 2 * d / 32 MFMA 16x16x32 (A = Q rows, B = K rows from LDS: both 16-byte
//      fragments along d), applies the sigmoid and the causal mask in fp32 and leaves P in LDS as T;
//   O: wave w owns CT 16-column tiles of the result for ALL row tiles, so that each V fragment (two transposed LDS reads of
//      four keys each) is read once per workgroup; one MFMA 16x16x32 per (row tile, column tile).
// The next tile's K and V rows are requested from global memory into registers before the current tile's products and
// stored to LDS after them.  A decode step's run has one token: row tiles without a valid row are skipped by whole waves.
// sm: Qs [64][d + 8] | Ks [32][d + 8] | Vs [32][dv + 8] | Ps [64][32 + 8]   (all T)
constexpr int SGM_ROWS = 64;
constexpr int SGM_MAXC = 4;      // 16-byte chunks of a K (V) tile per thread: d (dv) up to 256

template <typename T, int CT>
__global__ __launch_bounds__(256) void sigmoid_attention_mfma_kernel(SgArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smraw[];
  const int d = a.d, dv = a.dv;
  const int qld = d + 8, vld = dv + 8, pld = SG_KT + 8;
  T* Qs = reinterpret_cast<T*>(smraw);
  T* Ks = Qs + SGM_ROWS * qld;
  T* Vs = Ks + SG_KT * qld;
  T* Ps = Vs + SG_KT * vld;
  __shared__ int row_pos[SGM_ROWS];
  __shared__ float row_mul[SGM_ROWS], row_add[SGM_ROWS];
  const int rep = a.heads / a.kv_heads;
  const int HR = a.heads_per_tile;
  const int chunks = (rep + HR - 1) / HR;
  const int g = blockIdx.y / chunks, hc = blockIdx.y - g * chunks;
  const int split = blockIdx.z;
  // runs come in token order, so a sequence's later (longer) runs are listed last: take them first
  const unsigned bx = gridDim.x - 1 - blockIdx.x;
  const int64_t t0 = a.blocks != nullptr ? a.blocks[2 * bx] : bx;
  const int nt = a.blocks != nullptr ? a.blocks[2 * bx + 1] : 1;
  const int b = a.tok_req != nullptr ? a.tok_req[t0] : (int)t0;
  const int32_t* table = a.req_to_token + a.req_pool_indices[b] * a.req_to_token_stride;
  const int h0 = g * rep + hc * HR;
  const int nh = min(HR, rep - hc * HR);
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const T* q = (const T*)a.q;
  const int dch = d / 8, vch = dv / 8;           // 16-byte chunks per row
  const int live_rows = nt * HR;                 // rows at or past this hold no (token, head)
  for (int e = tid; e < SGM_ROWS * dch; e += 256) {
    const int r = e / dch, ch = e - r * dch;
    const int tl = r / HR, hl = r - tl * HR;
    Vec<T, 8> val;
    if (tl < nt && hl < nh) {
      val = ldvec<T, 8>(q + (t0 + tl) * a.q_token_stride + (int64_t)(h0 + hl) * a.q_head_stride + ch * 8);
    } else {
#pragma unroll
      for (int x = 0; x < 8; ++x) val.v[x] = from_f32<T>(0.f);
    }
    lds_store16(Qs + r * qld + ch * 8, val);
  }
  if (tid < SGM_ROWS) {
    const int tl = tid / HR, hl = tid - tl * HR;
    const bool ok = tl < nt && hl < nh;
    row_pos[tid] = ok ? (int)a.positions[t0 + tl] : -1;
    row_mul[tid] = ok ? a.scale * a.temp[h0 + hl] : 0.f;
    row_add[tid] = ok ? a.bias[h0 + hl] : 0.f;
  }
  const int last = (int)a.positions[t0 + nt - 1];
  const int tiles = last / SG_KT + 1;
  const int per = (tiles + a.num_splits - 1) / a.num_splits;
  const int tile_lo = split * per, tile_hi = min(tiles, tile_lo + per);
  const int nblk = dv / 16;
  f32x4 acc[4][CT];
#pragma unroll
  for (int rt = 0; rt < 4; ++rt)
#pragma unroll
    for (int c = 0; c < CT; ++c) acc[rt][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  const T* kc = (const T*)a.k_cache;
  const T* vc = (const T*)a.v_cache;
  using Frag = typename Mfma<T>::frag;
  Vec<T, 8> kreg[SGM_MAXC], vreg[SGM_MAXC];
  // Every load is unconditional (a load under a branch is waited for at the branch's end, one latency per load): chunk
  // numbers past the tile's last one are clamped to it -- all lanes then read one address -- and never stored.  The cache
  // slots of a tile's keys are read from the request table one tile before the rows themselves are requested, so that
  // a request does not start with a wait for its own addresses.
  int64_t ksrc[SGM_MAXC], vsrc[SGM_MAXC];
  auto load_slots = [&](int tile) {
    const int j0 = tile * SG_KT;
#pragma unroll
    for (int u = 0; u < SGM_MAXC; ++u) {
      const int ek = min(tid + 256 * u, SG_KT * dch - 1), ev = min(tid + 256 * u, SG_KT * vch - 1);
      const int kk = ek / dch, kv = ev / vch;
      // keys past the run's last one are masked below; any valid row will do
      ksrc[u] = ((int64_t)table[min(j0 + kk, last)] * a.kv_heads + g) * d + (ek - kk * dch) * 8;
      vsrc[u] = ((int64_t)table[min(j0 + kv, last)] * a.kv_heads + g) * dv + (ev - kv * vch) * 8;
    }
  };
  auto request = [&]() {
#pragma unroll
    for (int u = 0; u < SGM_MAXC; ++u) {
      kreg[u] = ldvec<T, 8>(kc + ksrc[u]);
      vreg[u] = ldvec<T, 8>(vc + vsrc[u]);
    }
  };
  if (tile_lo < tile_hi) {
    load_slots(tile_lo);
    request();
    load_slots(tile_lo + 1);
  }
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const int j0 = tile * SG_KT;
    __syncthreads();                             // the last tile's readers are done (and, the first time, Qs is written)
#pragma unroll
    for (int u = 0; u < SGM_MAXC; ++u) {
      const int e = tid + 256 * u;
      if (e < SG_KT * dch) {
        const int kk = e / dch, ch = e - kk * dch;
        lds_store16(Ks + kk * qld + ch * 8, kreg[u]);
      }
      if (e < SG_KT * vch) {
        const int kk = e / vch, ch = e - kk * vch;
        lds_store16(Vs + kk * vld + ch * 8, vreg[u]);
      }
    }
    __syncthreads();
    if (tile + 1 < tile_hi) {                    // in flight during this tile's products
      request();
      load_slots(tile + 2);
    }
    if (16 * wv < live_rows) {
      f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
      for (int c = 0; c < d; c += 32) {
        const Frag af = lds_load16<Frag>(Qs + (16 * wv + li) * qld + c + 8 * lg);
        const Frag b0 = lds_load16<Frag>(Ks + li * qld + c + 8 * lg);
        const Frag b1 = lds_load16<Frag>(Ks + (16 + li) * qld + c + 8 * lg);
        s0 = Mfma<T>::run(af, b0, s0);
        s1 = Mfma<T>::run(af, b1, s1);
      }
      // result lane: rows 16 wv + 4 lg + x, key columns li (s0) and 16 + li (s1)
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int r = 16 * wv + 4 * lg + x;
        const int rp = row_pos[r];
        const float m = row_mul[r], ad = row_add[r];
        lds_store2(Ps + r * pld + li, from_f32<T>(j0 + li <= rp ? sg_sigmoid_fast(s0[x] * m + ad) : 0.f));
        lds_store2(Ps + r * pld + 16 + li, from_f32<T>(j0 + 16 + li <= rp ? sg_sigmoid_fast(s1[x] * m + ad) : 0.f));
      }
    }
    __syncthreads();
    {
      // V fragments of this wave's column tiles: lane group lg supplies keys 8 lg .. 8 lg + 7 as two transposed reads
      const T* vrow = Vs + (8 * lg + (li >> 2)) * vld + 4 * (li & 3) + 16 * CT * wv;
      typename TrRead<T>::v4 lo[CT], hi[CT];
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        if (CT * wv + c < nblk) {
          lo[c] = TrRead<T>::run(vrow + 16 * c);
          hi[c] = TrRead<T>::run(vrow + 4 * vld + 16 * c);
        }
      }
#pragma unroll
      for (int rt = 0; rt < 4; ++rt) {
        if (16 * rt < live_rows) {
          const Frag pa = lds_load16<Frag>(Ps + (16 * rt + li) * pld + 8 * lg);
#pragma unroll
          for (int c = 0; c < CT; ++c) {
            if (CT * wv + c < nblk) {
              typename TrRead<T>::v4 both[2] = {lo[c], hi[c]};
              acc[rt][c] = Mfma<T>::run(pa, __builtin_bit_cast(Frag, both), acc[rt][c]);
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      if (CT * wv + c >= nblk) continue;
      const int col = 16 * (CT * wv + c) + li;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int r = 16 * rt + 4 * lg + x;
        const int tl = r / HR, hl = r - tl * HR;
        if (tl >= nt || hl >= nh) continue;
        if (a.num_splits > 1) {
          a.partial[(((int64_t)split * a.tokens + t0 + tl) * a.heads + h0 + hl) * dv + col] = acc[rt][c][x];
        } else {
          ((T*)a.out)[(t0 + tl) * a.out_token_stride + (int64_t)(h0 + hl) * a.out_head_stride + col] = from_f32<T>(acc[rt][c][x]);
        }
      }
    }
  }
}

inline bool sg_mfma_shape(int dtype, int d, int dv) {
  return dtype != MI355_F32 && d % 32 == 0 && dv % 16 == 0 && d <= 32 * SGM_MAXC * 2 && dv <= 32 * SGM_MAXC * 2;
}

template <typename T> int launch_sigmoid(const SgArgs& a, dim3 grid, bool mfma, hipStream_t stream) {
  if constexpr (!std::is_same<T, float>::value) {
    if (mfma) {
      const size_t lds = ((size_t)(SGM_ROWS + SG_KT) * (a.d + 8) + (size_t)SG_KT * (a.dv + 8) + SGM_ROWS * (SG_KT + 8)) * sizeof(T);
      const int nblk = a.dv / 16;
#define MI355_SG_LAUNCH(CT)                                                                                                    \
  do {                                                                                                                         \
    if (lds > 64 * 1024) {                                                                                                     \
      hipError_t e = hipFuncSetAttribute((const void*)sigmoid_attention_mfma_kernel<T, CT>,                                    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                                \
      MI355_REQUIRE(e == hipSuccess, MI355_ERR_LAUNCH, "sigmoid_attention: %zu bytes of LDS refused", lds);                    \
    }                                                                                                                          \
    hipLaunchKernelGGL((sigmoid_attention_mfma_kernel<T, CT>), grid, dim3(256), lds, stream, a);                               \
  } while (0)
      if (nblk <= 4) MI355_SG_LAUNCH(1);
      else if (nblk <= 8) MI355_SG_LAUNCH(2);
      else MI355_SG_LAUNCH(4);
#undef MI355_SG_LAUNCH
      return MI355_OK;
    }
  }
  const size_t lds = ((size_t)SG_ROWS * a.d + (size_t)SG_KT * (a.d + 1) + (size_t)SG_KT * a.dv + SG_ROWS * SG_KT) * sizeof(float);
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)sigmoid_attention_valu_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    MI355_REQUIRE(e == hipSuccess, MI355_ERR_LAUNCH, "sigmoid_attention: %zu bytes of LDS refused", lds);
  }
  hipLaunchKernelGGL((sigmoid_attention_valu_kernel<T>), grid, dim3(256), lds, stream, a);
  return MI355_OK;
}

inline int heads_per_tile(int heads, int kv_heads, int rows) { return std::min(heads / kv_heads, rows); }

}  // namespace
}  // namespace mi355

using namespace mi355;

int mi355_sigmoid_attention_block_tokens(int heads, int kv_heads, int head_dim, int v_head_dim, int dtype) {
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads) return 0;
  const int rows = sg_mfma_shape(dtype, head_dim, v_head_dim) ? SGM_ROWS : SG_ROWS;
  return std::max(1, rows / heads_per_tile(heads, kv_heads, rows));
}

int mi355_sigmoid_attention(void* out, const void* q, const void* k_cache, const void* v_cache, const int32_t* req_to_token,
                            const int64_t* req_pool_indices, const int32_t* tok_req, const int64_t* positions,
                            const int32_t* blocks, int64_t num_blocks, const float* temp, const float* bias,
                            int64_t q_token_stride, int64_t q_head_stride, int64_t out_token_stride, int64_t out_head_stride,
                            int64_t req_to_token_stride, int heads, int kv_heads, int head_dim, int v_head_dim, float scale,
                            int num_splits, float* split_scratch, int64_t tokens, int max_run, int dtype, void* stream) {
  MI355_REQUIRE(out && q && k_cache && v_cache && req_to_token && req_pool_indices && positions && temp && bias, MI355_ERR_INVALID,
                "sigmoid_attention: null pointer");
  MI355_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && head_dim > 0 && v_head_dim > 0 && tokens >= 0 &&
                    num_blocks >= 0, MI355_ERR_INVALID, "sigmoid_attention: bad shape");
  MI355_REQUIRE(head_dim <= 512 && v_head_dim <= 256, MI355_ERR_UNSUPPORTED, "sigmoid_attention: head width %d / %d not served",
                head_dim, v_head_dim);
  MI355_REQUIRE(num_splits >= 1 && num_splits <= 64 && (num_splits == 1 || (split_scratch && blocks == nullptr)), MI355_ERR_INVALID,
                "sigmoid_attention: key splits serve launches of one token per run and need scratch");
  MI355_REQUIRE(blocks != nullptr || num_blocks == tokens, MI355_ERR_INVALID, "sigmoid_attention: without runs, one block per token");
  if (num_blocks == 0) return MI355_OK;
  SgArgs a;
  a.out = out; a.partial = split_scratch; a.q = q; a.k_cache = k_cache; a.v_cache = v_cache; a.req_to_token = req_to_token;
  a.req_pool_indices = req_pool_indices; a.tok_req = tok_req; a.positions = positions; a.blocks = blocks; a.temp = temp;
  a.bias = bias; a.q_token_stride = q_token_stride; a.q_head_stride = q_head_stride; a.out_token_stride = out_token_stride;
  a.out_head_stride = out_head_stride; a.req_to_token_stride = req_to_token_stride; a.tokens = tokens; a.heads = heads;
  // the matrix-core kernel needs 16-byte rows everywhere; a caller whose q is laid out otherwise gets the vector-ALU kernel,
  // whose runs are shorter: max_run says how long the caller's runs may be, and a launch that cannot take them is refused
  const bool mfma = sg_mfma_shape(dtype, head_dim, v_head_dim) && q_token_stride % 8 == 0 && q_head_stride % 8 == 0 &&
                    aligned16(q) && aligned16(k_cache) && aligned16(v_cache);
  const int rows = mfma ? SGM_ROWS : SG_ROWS;
  a.kv_heads = kv_heads; a.d = head_dim; a.dv = v_head_dim; a.heads_per_tile = heads_per_tile(heads, kv_heads, rows);
  a.tokens_per_tile = std::max(1, rows / a.heads_per_tile); a.num_splits = num_splits; a.scale = scale;
  MI355_REQUIRE(max_run >= 1 && max_run <= a.tokens_per_tile, MI355_ERR_UNSUPPORTED,
                "sigmoid_attention: runs of up to %d tokens, this launch takes %d", max_run, a.tokens_per_tile);
  const int rep = heads / kv_heads;
  const int chunks = (rep + a.heads_per_tile - 1) / a.heads_per_tile;
  const dim3 grid((unsigned)num_blocks, (unsigned)(kv_heads * chunks), (unsigned)num_splits);
  MI355_REQUIRE(kv_heads * chunks <= 65535, MI355_ERR_UNSUPPORTED, "sigmoid_attention: too many heads");
  int rc = MI355_OK;
  MI355_DISPATCH_DTYPE(dtype, "sigmoid_attention", { rc = launch_sigmoid<T>(a, grid, mfma, (hipStream_t)stream); });
  if (rc != MI355_OK) return rc;
  MI355_CHECK_LAUNCH("sigmoid_attention");
  if (num_splits > 1) {
    const int64_t n = tokens * heads * v_head_dim;
    const int g2 = (int)std::min<int64_t>((n + 255) / 256, 4096);
    MI355_DISPATCH_DTYPE(dtype, "sigmoid_attention", {
      hipLaunchKernelGGL((sigmoid_attention_sum_kernel<T>), dim3(g2), dim3(256), 0, (hipStream_t)stream, (T*)out, split_scratch,
                         tokens, heads, v_head_dim, num_splits, out_token_stride, out_head_stride);
    });
    MI355_CHECK_LAUNCH("sigmoid_attention(sum)");
  }
  return MI355_OK;
}
