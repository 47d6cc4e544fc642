// Mixture-of-experts feed-forwards: ungated W_down gelu(W_up h), or gated
// W_down (act(W_gate h) * (W_up h)) with [gate rows | up rows] stacked in one weight per expert.
//
// moe_route_scores : softmax over all router outputs, the k largest of score + correction chosen,
//               weights = chosen scores / (their sum + 1e-20).
// epilogues of moe_gemm (ACT): 0 none, 1 erf-GELU, 2 tanh-GELU(gate) * up, 3 SiLU(gate) * up. In the
//               gated forms a workgroup's B tile holds matching gate and up columns, so the product is
//               formed in registers and only F columns are written.
// ids >= E (identity experts) get no tile: moe_group marks their pairs -1 and moe_combine adds
//               w * h for them.
//
// moe_route   : top-k of fp32 router logits (ties to the lower index), softmax over the chosen.
// moe_group   : one workgroup sorts the (token, choice) pairs by expert into 64-row tiles
//               (counts and ranks through LDS atomics; a tile holds rows of one expert only).
// moe_gemm    : tile GEMM, 64 rows x 64 columns per workgroup, K stepped by 16 through LDS,
//               4 x 4 outputs per thread, fp32 accumulation in a fixed K order (a row's sums do
//               not depend on its tile or on the rest of the step); optional erf-GELU epilogue.
// moe_combine : out[t] = sum_j w[t, j] * y[slot(t, j)] in fp32.
#include "seqmix_common.h"

using namespace sm;

namespace {

constexpr int TM = 64, TN = 64, TK = 16;

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int E, int k,
                                                        int* __restrict__ ids, float* __restrict__ w, int T,
                                                        int sigmoid) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + (int64_t)t * E;
  int* oi = ids + (int64_t)t * k;
  float* ow = w + (int64_t)t * k;
  for (int j = 0; j < k; ++j) {
    float best = -INFINITY;
    int bi = -1;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int i = 0; i < j; ++i) taken |= oi[i] == e;
      const float v = z[e];
      if (!taken && (bi < 0 || v > best)) {
        best = v;
        bi = e;
      }
    }
    oi[j] = bi;
    ow[j] = best;
  }
  if (sigmoid) {  // every chosen logit's own sigmoid
    for (int j = 0; j < k; ++j) ow[j] = 1.f / (1.f + expf(-ow[j]));
    return;
  }
  const float m = ow[0];  // the first chosen is the largest
  float s = 0.f;
  for (int j = 0; j < k; ++j) {
    const float p = expf(ow[j] - m);
    ow[j] = p;
    s += p;
  }
  for (int j = 0; j < k; ++j) ow[j] /= s;
}

// One wave per token, lanes over experts (E <= 512: up to 8 logits per lane in registers): k rounds
// of a wave-wide arg-max over the logits not yet chosen, ties to the lower index.
__global__ __launch_bounds__(256) void moe_route_wave_kernel(const float* __restrict__ logits, int E, int k,
                                                             int* __restrict__ ids, float* __restrict__ w, int T,
                                                             int sigmoid) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (t >= T) return;
  const float* z = logits + (int64_t)t * E;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < E ? z[e] : -INFINITY;
  }
  float m0 = 0.f, sum = 0.f, mine = 0.f;  // lane j keeps the j-th chosen weight
  int mine_id = 0;
  unsigned taken = 0;  // bit i: this lane's logit i is already chosen
  for (int j = 0; j < k; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = lane + 64 * i;
      if (e < E && !(taken >> i & 1u) && (bi == 0x7fffffff || v[i] > best)) {
        best = v[i];
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ob > best || (ob == best && oi < bi))) {
        best = ob;
        bi = oi;
      }
    }
    if (j == 0) m0 = best;
    const float p = sigmoid ? 1.f / (1.f + expf(-best)) : expf(best - m0);
    sum += p;
    if (lane == j) {
      mine = p;
      mine_id = bi;
    }
    if ((bi & 63) == lane) taken |= 1u << (bi >> 6);
  }
  if (lane < k) {
    ids[(int64_t)t * k + lane] = mine_id;
    w[(int64_t)t * k + lane] = sigmoid ? mine : mine / sum;
  }
}

// One wave per token, lanes over the router's outputs (E <= 512).
__global__ __launch_bounds__(256) void moe_route_scores_wave_kernel(const float* __restrict__ logits,
                                                                    const float* __restrict__ corr, int E, int k,
                                                                    int* __restrict__ ids, float* __restrict__ w,
                                                                    int T) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (t >= T) return;
  const float* z = logits + (int64_t)t * E;
  float v[8], sc[8];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < E ? z[e] : -INFINITY;
    mx = fmaxf(mx, v[i]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    sc[i] = lane + 64 * i < E ? expf(v[i] - mx) : 0.f;
    sum += sc[i];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = lane + 64 * i;
    sc[i] = sc[i] / sum;                            // the score
    v[i] = e < E ? sc[i] + corr[e] : -INFINITY;     // what the choice looks at
  }
  float wsum = 0.f, mine = 0.f;
  int mine_id = 0;
  unsigned taken = 0;
  for (int j = 0; j < k; ++j) {
    float best = -INFINITY, bs_ = 0.f;
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = lane + 64 * i;
      if (e < E && !(taken >> i & 1u) && (bi == 0x7fffffff || v[i] > best)) {
        best = v[i];
        bs_ = sc[i];
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64), os = __shfl_xor(bs_, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ob > best || (ob == best && oi < bi))) {
        best = ob;
        bs_ = os;
        bi = oi;
      }
    }
    wsum += bs_;
    if (lane == j) {
      mine = bs_;
      mine_id = bi;
    }
    if ((bi & 63) == lane) taken |= 1u << (bi >> 6);
  }
  if (lane < k) {
    ids[(int64_t)t * k + lane] = mine_id;
    w[(int64_t)t * k + lane] = mine / (wsum + 1e-20f);
  }
}

// Any E: one thread per token.
__global__ __launch_bounds__(256) void moe_route_scores_kernel(const float* __restrict__ logits,
                                                               const float* __restrict__ corr, int E, int k,
                                                               int* __restrict__ ids, float* __restrict__ w, int T) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + (int64_t)t * E;
  int* oi = ids + (int64_t)t * k;
  float* ow = w + (int64_t)t * k;
  float mx = -INFINITY, sum = 0.f;
  for (int e = 0; e < E; ++e) mx = fmaxf(mx, z[e]);
  for (int e = 0; e < E; ++e) sum += expf(z[e] - mx);
  float wsum = 0.f;
  for (int j = 0; j < k; ++j) {
    float best = -INFINITY, bsc = 0.f;
    int bi = -1;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int i = 0; i < j; ++i) taken |= oi[i] == e;
      const float sc = expf(z[e] - mx) / sum;
      const float c = sc + corr[e];
      if (!taken && (bi < 0 || c > best)) {
        best = c;
        bsc = sc;
        bi = e;
      }
    }
    oi[j] = bi;
    ow[j] = bsc;
    wsum += bsc;
  }
  for (int j = 0; j < k; ++j) ow[j] /= (wsum + 1e-20f);
}

__global__ __launch_bounds__(1024) void moe_group_kernel(const int* __restrict__ ids, int n, int E,
                                                         int* __restrict__ slot_row, int* __restrict__ tile_e,
                                                         int* __restrict__ pair_slot, int max_tiles) {
  extern __shared__ int sh[];  // cnt[E] | first_tile[E]
  int* cnt = sh;
  int* first = sh + E;
  for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
  for (int i = threadIdx.x; i < max_tiles * TM; i += 1024) slot_row[i] = -1;
  for (int i = threadIdx.x; i < max_tiles; i += 1024) tile_e[i] = -1;
  __syncthreads();
  for (int p = threadIdx.x; p < n; p += 1024)
    if (ids[p] < E) atomicAdd(&cnt[ids[p]], 1);  // ids >= E: identity experts, no tile
  __syncthreads();
  if (threadIdx.x == 0) {
    int tile = 0;
    for (int e = 0; e < E; ++e) {
      first[e] = tile;
      const int nt = (cnt[e] + TM - 1) / TM;
      for (int i = 0; i < nt; ++i) tile_e[tile + i] = e;
      tile += nt;
      cnt[e] = 0;  // reused as the running rank
    }
  }
  __syncthreads();
  for (int p = threadIdx.x; p < n; p += 1024) {
    const int e = ids[p];
    if (e >= E) {
      pair_slot[p] = -1;
      continue;
    }
    const int slot = first[e] * TM + atomicAdd(&cnt[e], 1);
    slot_row[slot] = p;
    pair_slot[p] = slot;
  }
}

// C[slot, n] = act(sum_k A[row(slot), k] * W[e, n, k]);  row(slot) = pair / kdiv (gathered
// tokens) when kdiv > 0, the slot itself otherwise.
__device__ __forceinline__ float gelu_erf_(float v) { return 0.5f * v * (1.f + erff(v * 0.70710678118654752f)); }
__device__ __forceinline__ float gelu_tanh_(float v) {
  return 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
}
template <int ACT>
__device__ __forceinline__ float gate_act_(float g) {
  return ACT == 2 ? gelu_tanh_(g) : g / (1.f + expf(-g));
}

// Gated forms (ACT >= 2): N is the number of OUTPUT columns F; the weight has 2 N rows [gate | up].
// The workgroup's 64 B rows are 32 gate rows n0.. and the 32 matching up rows; a thread's four
// columns are two gate columns and their two up columns.
template <typename T, int ACT>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const T* __restrict__ A, int64_t a_stride, int kdiv,
                                                       const int* __restrict__ slot_row,
                                                       const int* __restrict__ tile_e, const T* __restrict__ Wt,
                                                       int N, int K, T* __restrict__ Cout,
                                                       const float* __restrict__ row_w) {
  const int e = tile_e[blockIdx.x];
  if (e < 0) return;
  __shared__ float sA[TK][TM + 4], sB[TK][TN + 4];
  __shared__ int srow[TM];
  __shared__ float sw[TM];  // the row's input weight (gated forms with row_w): scales both sums
  const int tid = threadIdx.x;
  constexpr bool GATED = ACT >= 2;
  const int slot0 = blockIdx.x * TM, n0 = blockIdx.y * (GATED ? TN / 2 : TN);
  if (tid < TM) {
    const int p = slot_row[slot0 + tid];
    srow[tid] = p < 0 ? -1 : (kdiv > 0 ? p / kdiv : slot0 + tid);
    sw[tid] = (row_w != nullptr && p >= 0) ? row_w[p] : 1.f;
  }
  __syncthreads();
  const T* We = Wt + (int64_t)e * (GATED ? 2 * N : N) * K;
  const int lr = tid >> 2, lk = (tid & 3) * 4;  // loader: row / column lr, 4 consecutive k
  const int ty = tid >> 4, tx = tid & 15;       // compute: rows ty*4.., columns tx*4.. (gated: see above)
  float acc[4][4] = {};
  const int arow = srow[lr];
  const int bcol = GATED ? n0 + (lr & 31) : n0 + lr;          // output column this B row belongs to
  const int brow = GATED && lr >= 32 ? N + bcol : bcol;         // its row in the expert's weight
  for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int kk = k0 + lk + i;
      sA[lk + i][lr] = (arow >= 0 && kk < K) ? ld(A + (int64_t)arow * a_stride + kk) : 0.f;
      sB[lk + i][lr] = (bcol < N && kk < K) ? ld(We + (int64_t)brow * K + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] = sA[kk][ty * 4 + i];
        b[i] = GATED ? sB[kk][(i >> 1) * 32 + tx * 2 + (i & 1)] : sB[kk][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (srow[r] < 0) continue;
    if (GATED) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int n = n0 + tx * 2 + j;
        if (n < N) st(Cout + (int64_t)(slot0 + r) * N + n, gate_act_<ACT>(sw[r] * acc[i][j]) * (sw[r] * acc[i][j + 2]));
      }
      continue;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (ACT == 1) v = gelu_erf_(v);
      st(Cout + (int64_t)(slot0 + r) * N + n, v);
    }
  }
}


// bf16 on the matrix cores: 64 rows x 128 columns per workgroup, K stepped by 64 through LDS
// (next step's global loads in flight during the MFMAs). Wave (wm, wn) owns rows 32 wm.. and
// columns 64 wn.. as 2 x 4 fragments of v_mfma_f32_16x16x32_bf16; fp32 accumulation in a fixed
// K order. Needs K % 8 == 0 and 16-byte aligned rows (vector loads).
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int MBK = 64, MLS = MBK + 8;  // LDS row stride 144 B

// NJ = 16-column fragments per wave: the workgroup's tile is 64 rows x MBN = 32 NJ columns
// (128 for steps with few rows per expert: more workgroups stream the weights; 256 for prompt-sized
// steps: twice the MFMAs per LDS pass and barrier).
// Gated forms (ACT >= 2): a wave's first NJ / 2 fragments are gate columns, the other NJ / 2 the
// matching up columns; the workgroup writes 16 NJ output columns.
template <int ACT, int NJ>
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(const bf16_t* __restrict__ A, int64_t a_stride, int kdiv,
                                                            const int* __restrict__ slot_row,
                                                            const int* __restrict__ tile_e,
                                                            const bf16_t* __restrict__ Wt, int N, int K,
                                                            bf16_t* __restrict__ Cout,
                                                            const float* __restrict__ row_w) {
  const int e = tile_e[blockIdx.x];
  if (e < 0) return;
  constexpr bool GATED = ACT >= 2;
  constexpr int MBN = 32 * NJ, NB = MBN / 32;  // NB = B chunks per thread and K step
  __shared__ __attribute__((aligned(16))) bf16_t sA[TM * MLS];
  __shared__ __attribute__((aligned(16))) bf16_t sB[MBN * MLS];
  __shared__ int srow[TM];
  __shared__ float sw[TM];  // the row's input weight (gated forms with row_w): scales both sums
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int slot0 = blockIdx.x * TM, n0 = blockIdx.y * (GATED ? MBN / 2 : MBN);
  if (tid < TM) {
    const int p = slot_row[slot0 + tid];
    srow[tid] = p < 0 ? -1 : (kdiv > 0 ? p / kdiv : slot0 + tid);
    sw[tid] = (row_w != nullptr && p >= 0) ? row_w[p] : 1.f;
  }
  __syncthreads();
  const bf16_t* We = Wt + (int64_t)e * (GATED ? 2 * N : N) * K;
  // LDS row r of the B tile -> (output column, weight row)
  auto bcol = [&](int r) {
    if (!GATED) return n0 + r;
    const int w = r / (16 * NJ), jj = (r % (16 * NJ)) / 16, c = r & 15;
    return n0 + w * 8 * NJ + (jj % (NJ / 2)) * 16 + c;
  };
  auto brow = [&](int r, int col) { return GATED && (r % (16 * NJ)) / 16 >= NJ / 2 ? N + col : col; };
  // staging: A 64 rows x 8 chunks of 16 B (2 per thread), B MBN x 8 (NB per thread)
  u32x4_t ra[2], rb[NB];
  auto load = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = tid + 256 * i, r = c >> 3, ch = c & 7;
      u32x4_t v = {0, 0, 0, 0};
      const int ar = srow[r];
      if (ar >= 0 && k0 + ch * 8 < K) v = *reinterpret_cast<const u32x4_t*>(A + (int64_t)ar * a_stride + k0 + ch * 8);
      ra[i] = v;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int c = tid + 256 * i, r = c >> 3, ch = c & 7;
      u32x4_t v = {0, 0, 0, 0};
      const int col = bcol(r);
      if (col < N && k0 + ch * 8 < K) v = *reinterpret_cast<const u32x4_t*>(We + (int64_t)brow(r, col) * K + k0 + ch * 8);
      rb[i] = v;
    }
  };
  auto store = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = tid + 256 * i;
      *reinterpret_cast<u32x4_t*>(&sA[(c >> 3) * MLS + (c & 7) * 8]) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int c = tid + 256 * i;
      *reinterpret_cast<u32x4_t*>(&sB[(c >> 3) * MLS + (c & 7) * 8]) = rb[i];
    }
  };
  f32x4_t acc[2][NJ];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int r16 = lane & 15, kq = lane >> 4;
  const int nk = (K + MBK - 1) / MBK;
  load(0);
  for (int kt = 0; kt < nk; ++kt) {
    __syncthreads();  // the previous step's fragments are read
    store();
    __syncthreads();
    if (kt + 1 < nk) load((kt + 1) * MBK);
#pragma unroll
    for (int ks = 0; ks < MBK / 32; ++ks) {
      bf16x8_t af[2], bfr[NJ];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        af[i] = *reinterpret_cast<const bf16x8_t*>(&sA[(wm * 32 + i * 16 + r16) * MLS + ks * 32 + kq * 8]);
#pragma unroll
      for (int j = 0; j < NJ; ++j)
        bfr[j] = *reinterpret_cast<const bf16x8_t*>(&sB[(wn * 16 * NJ + j * 16 + r16) * MLS + ks * 32 + kq * 8]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
  }
  // acc[i][j][r] = C[row 32 wm + 16 i + 4 kq + r][column 16 NJ wn + 16 j + r16]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = wm * 32 + i * 16 + kq * 4 + r;
      if (srow[row] < 0) continue;
      if (GATED) {
#pragma unroll
        for (int j = 0; j < NJ / 2; ++j) {
          const int n = n0 + wn * 8 * NJ + j * 16 + r16;
          if (n < N)
            st(Cout + (int64_t)(slot0 + row) * N + n,
               gate_act_<ACT>(sw[row] * acc[i][j][r]) * (sw[row] * acc[i][j + NJ / 2][r]));
        }
        continue;
      }
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int n = n0 + wn * 16 * NJ + j * 16 + r16;
        if (n >= N) continue;
        float v = acc[i][j][r];
        if (ACT == 1) v = gelu_erf_(v);
        st(Cout + (int64_t)(slot0 + row) * N + n, v);
      }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const T* __restrict__ y, const int* __restrict__ pair_slot,
                                                          const float* __restrict__ w, int k, int d,
                                                          T* __restrict__ out, const T* __restrict__ h) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < d; c += 256) {
    float s = 0.f;
    for (int j = 0; j < k; ++j) {
      const int slot = pair_slot[t * k + j];
      // slot < 0: an identity expert returns the token's own input
      s += (w ? w[t * k + j] : 1.f) * (slot >= 0 ? ld(y + (int64_t)slot * d + c) : ld(h + t * d + c));
    }
    st(out + t * d + c, s);
  }
}

// bf16 rows that are 16-byte multiples: a thread sums eight columns from 16-byte loads.
__global__ __launch_bounds__(256) void moe_combine_vec_kernel(const bf16_t* __restrict__ y,
                                                              const int* __restrict__ pair_slot,
                                                              const float* __restrict__ w, int k, int d,
                                                              bf16_t* __restrict__ out, const bf16_t* __restrict__ h) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x * 8; c < d; c += 256 * 8) {
    float s[8] = {};
    for (int j = 0; j < k; ++j) {
      const int slot = pair_slot[t * k + j];
      const float wj = w ? w[t * k + j] : 1.f;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(slot >= 0 ? y + (int64_t)slot * d + c : h + t * d + c);
#pragma unroll
      for (int q = 0; q < 8; ++q) s[q] += wj * __uint_as_float((v[q >> 1] >> (16 * (q & 1))) << 16);
    }
    u32x4_t o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const __bf16 a = (__bf16)s[2 * q], b = (__bf16)s[2 * q + 1];
      o[q] = (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
    }
    *reinterpret_cast<u32x4_t*>(out + t * d + c) = o;
  }
}

}  // namespace

extern "C" {

// sigmoid: the weights are the chosen logits' sigmoids instead of the softmax over the chosen logits.
void sm_moe_route(const float* logits, int E, int k, int* ids, float* w, int T, int sigmoid, hipStream_t stream) {
  if (T == 0) return;
  if (E <= 512 && k <= 64) {
    hipLaunchKernelGGL(moe_route_wave_kernel, dim3((T + 3) / 4), dim3(256), 0, stream, logits, E, k, ids, w, T,
                       sigmoid);
    return;
  }
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + 255) / 256), dim3(256), 0, stream, logits, E, k, ids, w, T, sigmoid);
}

void sm_moe_route_scores(const float* logits, const float* corr, int E, int k, int* ids, float* w, int T,
                         hipStream_t stream) {
  if (T == 0) return;
  if (E <= 512 && k <= 64) {
    hipLaunchKernelGGL(moe_route_scores_wave_kernel, dim3((T + 3) / 4), dim3(256), 0, stream, logits, corr, E, k, ids,
                       w, T);
    return;
  }
  hipLaunchKernelGGL(moe_route_scores_kernel, dim3((T + 255) / 256), dim3(256), 0, stream, logits, corr, E, k, ids, w,
                     T);
}

void sm_moe_group(const int* ids, int n, int E, int* slot_row, int* tile_e, int* pair_slot, int max_tiles,
                  hipStream_t stream) {
  hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), 2 * E * sizeof(int), stream, ids, n, E, slot_row, tile_e,
                     pair_slot, max_tiles);
}

// act: 0 none, 1 erf-GELU, 2 tanh-GELU(gate) * up, 3 SiLU(gate) * up. N = output columns (the gated
// forms read a weight of 2 N rows per expert).
// row_w (gated forms): fp32 weight per (token, choice) pair that scales the row's INPUT, applied to
// both fp32 sums before the activation; nullptr = 1.
void sm_moe_gemm(const void* A, int64_t a_stride, int kdiv, const int* slot_row, const int* tile_e, const void* W,
                 int N, int K, void* C, int max_tiles, int rows_hint, int act, int f32, const float* row_w,
                 hipStream_t stream) {
  const bool gated = act >= 2;
  if (!f32 && K % 8 == 0 && a_stride % 8 == 0 && ((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0) {
    // wide tiles when the step has prompt-sized row counts (most tiles are full) and N is wide
    const bool wide = N >= 256 && rows_hint >= 32 * max_tiles;
    const int mbn = (wide ? 256 : 128) / (gated ? 2 : 1);
    const dim3 g2(max_tiles, (N + mbn - 1) / mbn);
#define SM_MF(A_, NJ)                                                                                          \
  hipLaunchKernelGGL((moe_gemm_mfma_kernel<A_, NJ>), g2, dim3(256), 0, stream, (const bf16_t*)A, a_stride, kdiv, \
                     slot_row, tile_e, (const bf16_t*)W, N, K, (bf16_t*)C, row_w)
#define SM_MF2(A_) \
  if (wide) SM_MF(A_, 8); \
  else SM_MF(A_, 4)
    if (act == 0) { SM_MF2(0); }
    else if (act == 1) { SM_MF2(1); }
    else if (act == 2) { SM_MF2(2); }
    else { SM_MF2(3); }
#undef SM_MF2
#undef SM_MF
    return;
  }
  const int tn = gated ? TN / 2 : TN;
  const dim3 grid(max_tiles, (N + tn - 1) / tn);
#define SM_GO(TYPE, A_)                                                                                         \
  hipLaunchKernelGGL((moe_gemm_kernel<TYPE, A_>), grid, dim3(256), 0, stream, (const TYPE*)A, a_stride, kdiv,   \
                     slot_row, tile_e, (const TYPE*)W, N, K, (TYPE*)C, row_w)
#define SM_GO2(TYPE)                   \
  if (act == 0) SM_GO(TYPE, 0);        \
  else if (act == 1) SM_GO(TYPE, 1);   \
  else if (act == 2) SM_GO(TYPE, 2);   \
  else SM_GO(TYPE, 3)
  if (f32) { SM_GO2(float); }
  else { SM_GO2(bf16_t); }
#undef SM_GO2
#undef SM_GO
}

void sm_moe_combine(const void* y, const int* pair_slot, const float* w, int k, int d, void* out, const void* h, int T,
                    int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL((moe_combine_kernel<float>), dim3(T), dim3(256), 0, stream, (const float*)y, pair_slot, w, k, d,
                       (float*)out, (const float*)h);
  else if (d % 8 == 0 && (((uintptr_t)y | (uintptr_t)out | (uintptr_t)h) & 15) == 0)
    hipLaunchKernelGGL(moe_combine_vec_kernel, dim3(T), dim3(256), 0, stream, (const bf16_t*)y, pair_slot, w, k, d,
                       (bf16_t*)out, (const bf16_t*)h);
  else
    hipLaunchKernelGGL((moe_combine_kernel<bf16_t>), dim3(T), dim3(256), 0, stream, (const bf16_t*)y, pair_slot, w, k,
                       d, (bf16_t*)out, (const bf16_t*)h);
}

}  // extern "C"
