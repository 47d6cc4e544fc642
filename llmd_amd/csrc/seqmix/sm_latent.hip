// Latent attention of any size over a paged latent cache (one row [latent R | rotated key dr]
// per token, shared by all heads).
//
// latent_rope_cache: rotate the query's rotary part (pairs (i, i + rot_dims/2) or (2i, 2i+1) over
//   the first rot_dims dimensions, angles from an fp32 cos/sin table) into the absorbed query, RMS-norm
//   the latent with its plain weight, rotate the shared key part and write the cache row. A layer
//   that reads another layer's cache passes no kv and rotates its queries only.
// All attention forms take an optional gate [T, H]: head h's result times sigmoid(gate[t, h]).
// latent_attention: one workgroup = QT consecutive token rows x 4 heads (one wave per head).
//   Keys stream through LDS in tiles of KT rows (fp32) shared by all 4 x QT (row, head) pairs;
//   a lane scores one key (dot over R + dr from LDS), the wave keeps an online softmax per pair,
//   and the lanes then own output columns for the P x latent product. Scores, softmax and the
//   accumulators are fp32. A row's result depends only on its own keys and the fixed tile
//   size, never on what else is in the step.
#include "seqmix_common.h"

using namespace sm;

namespace {

constexpr int NT = 256;

template <typename T>
__global__ __launch_bounds__(NT) void latent_rope_cache_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ kv, int64_t kv_stride,
    const T* __restrict__ norm_w, float eps, const int64_t* __restrict__ positions,
    const float* __restrict__ cos_sin, int H, int dn, int dr, int rot_dims, int R,
    const int64_t* __restrict__ slots, T* __restrict__ cache, T* __restrict__ q_abs, int interleaved) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int half = rot_dims >> 1;
  const float* cs = cos_sin + positions[t] * rot_dims;  // [cos(half) | sin(half)]
  const int Dk = R + dr;
  // element i of a rotated vector at src
  auto rot = [&](const T* src, int i) {
    if (i >= rot_dims) return ld(src + i);
    if (interleaved) {
      const int f = i >> 1;
      return (i & 1) ? ld(src + i) * cs[f] + ld(src + i - 1) * cs[half + f]
                     : ld(src + i) * cs[f] - ld(src + i + 1) * cs[half + f];
    }
    return i < half ? ld(src + i) * cs[i] - ld(src + i + half) * cs[half + i]
                    : ld(src + i) * cs[i - half] + ld(src + i - half) * cs[i];
  };
  // query: rotary part of every head -> q_abs[t, h, R + i]
  for (int e = threadIdx.x; e < H * dr; e += NT) {
    const int h = e / dr, i = e - h * dr;
    st(q_abs + (t * H + h) * Dk + R + i, rot(q + t * q_stride + (int64_t)h * (dn + dr) + dn, i));
  }
  if (kv == nullptr) return;
  // latent: RMS norm with a plain weight
  const T* kr = kv + t * kv_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < R; c += NT) {
    const float v = ld(kr + c);
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const float inv = 1.f / sqrtf(ss / (float)R + eps);
  T* row = cache + slot * Dk;
  for (int c = threadIdx.x; c < R; c += NT) st(row + c, ld(kr + c) * inv * ld(norm_w + c));
  for (int i = threadIdx.x; i < dr; i += NT) st(row + R + i, rot(kr + R, i));
}

// RC = ceil(R / 64) output columns per lane; QT token rows per workgroup.
template <typename T, int RC, int QT>
__global__ __launch_bounds__(NT) void latent_attention_kernel(
    const T* __restrict__ q_abs, const T* __restrict__ cache, const int* __restrict__ tables, int W, int bs,
    const int* __restrict__ row_seq, const int* __restrict__ row_len, float scale, int H, int R, int Dk, int KT,
    int T_rows, T* __restrict__ out, const T* __restrict__ gate, int64_t gate_stride) {
  extern __shared__ float lds[];
  const int KS = Dk + 1;                 // key row stride in LDS (odd: lanes hit distinct banks)
  float* sK = lds;                       // [KT][KS]
  float* sQ = lds + KT * KS;             // [QT][4][Dk], pre-scaled
  const int t0 = blockIdx.x * QT;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * 4 + wave;
  const bool head_ok = h < H;

  for (int e = threadIdx.x; e < QT * 4 * Dk; e += NT) {
    const int r = e / (4 * Dk), rem = e - r * 4 * Dk;
    const int w = rem / Dk, d = rem - w * Dk;
    const int t = t0 + r, hh = blockIdx.y * 4 + w;
    sQ[e] = (t < T_rows && hh < H) ? ld(q_abs + ((int64_t)t * H + hh) * Dk + d) * scale : 0.f;
  }

  int seq_r[QT], len_r[QT];
  bool done[QT];
#pragma unroll
  for (int r = 0; r < QT; ++r) {
    const int t = t0 + r;
    done[r] = t >= T_rows;
    seq_r[r] = done[r] ? -1 : row_seq[t];
    len_r[r] = done[r] ? 0 : row_len[t];
  }

  for (int pass = 0; pass < QT; ++pass) {
    // rows of this pass: those of the first unfinished row's sequence
    int seq = -1;
#pragma unroll
    for (int r = 0; r < QT; ++r)
      if (seq < 0 && !done[r]) seq = seq_r[r];
    if (seq < 0) break;
    bool act[QT];
    int maxlen = 0;
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      act[r] = !done[r] && seq_r[r] == seq;
      if (act[r]) maxlen = max(maxlen, len_r[r]);
    }
    float m[QT], l[QT], acc[QT][RC];
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      m[r] = -INFINITY;
      l[r] = 0.f;
#pragma unroll
      for (int c = 0; c < RC; ++c) acc[r][c] = 0.f;
    }
    const int* bt = tables + (int64_t)seq * W;
    for (int k0 = 0; k0 < maxlen; k0 += KT) {
      __syncthreads();  // previous tile fully used (and sQ written, first time)
      for (int e = threadIdx.x; e < KT * Dk; e += NT) {
        const int j = e / Dk, d = e - j * Dk;
        const int key = k0 + j;
        float v = 0.f;
        if (key < maxlen) {
          const int64_t rowi = (int64_t)bt[key / bs] * bs + (key % bs);
          v = ld(cache + rowi * Dk + d);
        }
        sK[j * KS + d] = v;
      }
      __syncthreads();
      if (!head_ok) continue;
#pragma unroll
      for (int r = 0; r < QT; ++r) {
        if (!act[r] || k0 >= len_r[r]) continue;
        const bool valid = lane < KT && k0 + lane < len_r[r];
        float s = -INFINITY;
        if (valid) {
          const float* qv = sQ + (r * 4 + wave) * Dk;
          const float* kr = sK + lane * KS;
          float a = 0.f;
          for (int d = 0; d < Dk; ++d) a += qv[d] * kr[d];
          s = a;
        }
        const float mn = fmaxf(m[r], wave_max(s));
        const float corr = expf(m[r] - mn);  // exp(-inf) = 0 on the first tile
        const float p = valid ? expf(s - mn) : 0.f;
        l[r] = l[r] * corr + wave_sum(p);
        m[r] = mn;
#pragma unroll
        for (int c = 0; c < RC; ++c) acc[r][c] *= corr;
        const int nk = min(KT, len_r[r] - k0);
        for (int j = 0; j < nk; ++j) {
          const float pj = __shfl(p, j, 64);
          const float* kr = sK + j * KS;
#pragma unroll
          for (int c = 0; c < RC; ++c) {
            const int col = lane + 64 * c;
            if (col < R) acc[r][c] += pj * kr[col];
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      if (!act[r]) continue;
      done[r] = true;
      if (!head_ok) continue;
      float inv = 1.f / l[r];
      if (gate) inv *= 1.f / (1.f + expf(-ld(gate + (int64_t)(t0 + r) * gate_stride + h)));
#pragma unroll
      for (int c = 0; c < RC; ++c) {
        const int col = lane + 64 * c;
        if (col < R) st(out + ((int64_t)(t0 + r) * H + h) * R + col, acc[r][c] * inv);
      }
    }
  }
}


// ---------------------------------------------------------------------------------------------
// bf16 form on the matrix cores. A workgroup takes one work item: up to 64 (token, head) rows of
// ONE sequence (consecutive tokens x all heads), 16 rows per wave. Keys stream through LDS in tiles
// of 32: the tile row-major for the scores (S^T = K Q^T, v_mfma_f32_16x16x32_bf16, fp32
// accumulation of exact bf16 products) and the latent part transposed for P x latent. Softmax is
// fp32 per row; the weights P enter the second product as a bf16 pair (hi + lo, two MFMAs), which
// keeps 16 mantissa bits of the fp32 weight. DkP = 32 NKS >= Dk and RP = 16 NCB >= R are the
// padded sizes (zeros in LDS and in the query fragments).
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int MKT = 32;  // keys per tile

template <int NKS, int NCB>
__global__ __launch_bounds__(NT) void latent_attention_mfma_kernel(
    const bf16_t* __restrict__ q_abs, const bf16_t* __restrict__ cache, const int* __restrict__ tables, int W, int bs,
    const int* __restrict__ items, const int* __restrict__ row_len, float scale, int H, int R, int Dk,
    bf16_t* __restrict__ out, int split_keys, float* __restrict__ part_o, float* __restrict__ part_ml,
    const bf16_t* __restrict__ gate, int64_t gate_stride) {
  constexpr int DkP = 32 * NKS, RP = 16 * NCB;
  constexpr int KS = DkP + 8, VS = MKT + 8, PS = MKT + 8;  // LDS row strides (bf16), 16-byte multiples
  // The weights P live in the key tile's space once the scores are done (one more barrier per
  // tile) when the tile is large enough: the largest form then needs 78 KB of LDS and two
  // workgroups share a CU, one staging its tile while the other multiplies.
  constexpr bool ALIAS = MKT * KS >= 2 * 4 * 16 * PS;
  __shared__ __attribute__((aligned(16))) bf16_t sK[MKT * KS];
  __shared__ __attribute__((aligned(16))) bf16_t sVt[RP * VS];
  __shared__ __attribute__((aligned(16))) bf16_t sP[ALIAS ? 8 : 2 * 4 * 16 * PS];
  bf16_t* const sPh = ALIAS ? sK : sP;
  bf16_t* const sPl = sPh + 4 * 16 * PS;
  const int seq = items[blockIdx.x * 3], tok0 = items[blockIdx.x * 3 + 1], ntok = items[blockIdx.x * 3 + 2];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, kq = lane >> 4;
  // this lane's query row (as the B operand's column): item row 16 wave + r16
  const int myrow = wave * 16 + r16;
  const bool row_ok = myrow < ntok * H;
  const int mytok = tok0 + (row_ok ? myrow / H : 0), myhead = row_ok ? myrow % H : 0;
  const int mylen = row_ok ? row_len[mytok] : 0;
  const int maxlen = row_len[tok0 + ntok - 1];  // the run's last token sees the most keys

  bf16x8_t qf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = ks * 32 + kq * 8 + i;
      const bf16_t w = (row_ok && d < Dk) ? q_abs[((int64_t)mytok * H + myhead) * Dk + d] : (bf16_t)0;
      qf[ks][i] = __builtin_bit_cast(__bf16, w);
    }
  }
  f32x4_t o[NCB];
#pragma unroll
  for (int n = 0; n < NCB; ++n) o[n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int* bt = tables + (int64_t)seq * W;
  bf16_t* ph = sPh + wave * 16 * PS;
  bf16_t* pl = sPl + wave * 16 * PS;
  const bool vec = (Dk & 7) == 0;

  // decode steps split a row's keys over blockIdx.y: this workgroup takes [kbeg, kend)
  const int nsplit = gridDim.y;
  const int kbeg = nsplit > 1 ? blockIdx.y * split_keys : 0;
  const int kend = nsplit > 1 ? min(maxlen, kbeg + split_keys) : maxlen;
  for (int k0 = kbeg; k0 < kend; k0 += MKT) {
    __syncthreads();  // the previous tile is no longer read
    // The tile's 16-byte chunks are all requested before any of them is used: one memory latency
    // per tile, not one per chunk. A tile lies inside one page when the page size is a multiple of
    // the tile (tiles start at multiples of 32 keys), so its block-table entry is read once.
    // Consecutive lanes take consecutive keys of one 8-column chunk: the transposed 2-byte writes
    // then fall into consecutive LDS words (chunk-major lanes would all hit one bank).
    constexpr int CPR = DkP / 8;                    // chunks per key row
    constexpr int NCH = (MKT * CPR + NT - 1) / NT;  // chunks per thread
    const bool one_page = (bs % MKT) == 0;
    const int64_t row0 = one_page ? (int64_t)bt[k0 / bs] * bs + (k0 % bs) : 0;
    u32x4_t pre[NCH];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int e = threadIdx.x + i * NT;
      const int c = e / MKT, j = e - c * MKT;
      const int key = k0 + j;
      u32x4_t v = {0, 0, 0, 0};
      if (e < MKT * CPR && key < kend && c * 8 < Dk) {
        const int64_t row = one_page ? row0 + j : (int64_t)bt[key / bs] * bs + (key % bs);
        const bf16_t* src = cache + row * Dk + c * 8;
        if (vec && c * 8 + 8 <= Dk) {
          v = *reinterpret_cast<const u32x4_t*>(src);
        } else {
#pragma unroll
          for (int q = 0; q < 8; ++q)
            if (c * 8 + q < Dk) v[q >> 1] |= (uint32_t)src[q] << (16 * (q & 1));
        }
      }
      pre[i] = v;
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int e = threadIdx.x + i * NT;
      if (e >= MKT * CPR) continue;
      const int c = e / MKT, j = e - c * MKT;
      *reinterpret_cast<u32x4_t*>(&sK[j * KS + c * 8]) = pre[i];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const int d = c * 8 + q;
        const bf16_t val = (bf16_t)(pre[i][q >> 1] >> (16 * (q & 1)));
        if (d < RP) sVt[d * VS + j] = d < R ? val : (bf16_t)0;
      }
    }
    __syncthreads();
    // scores of this lane's row against keys k0 + 16 kb + 4 kq + r
    float sc[2][4];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      f32x4_t a = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const bf16x8_t ka = *reinterpret_cast<const bf16x8_t*>(&sK[(kb * 16 + r16) * KS + ks * 32 + kq * 8]);
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[ks], a, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
        sc[kb][r] = (k0 + kb * 16 + kq * 4 + r < min(mylen, kend)) ? a[r] * scale : -INFINITY;
    }
    if (ALIAS) __syncthreads();  // every wave has read its keys: their space takes the weights
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, sc[kb][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    const float mref = (mn == -INFINITY) ? 0.f : mn;  // a row with no key yet
    const float corr = expf(m - mref);
    float psum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float pv = expf(sc[kb][r] - mref);
        psum += pv;
        const __bf16 hi = (__bf16)pv;
        const __bf16 lo = (__bf16)(pv - (float)hi);
        ph[r16 * PS + kb * 16 + kq * 4 + r] = __builtin_bit_cast(bf16_t, hi);
        pl[r16 * PS + kb * 16 + kq * 4 + r] = __builtin_bit_cast(bf16_t, lo);
      }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    m = mn;
    // the accumulators hold rows 4 kq + r: their correction comes from the lane that owns the row
    float cr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) cr[r] = __shfl(corr, kq * 4 + r, 64);
    __syncthreads();  // P of every wave is in LDS
    const bf16x8_t pah = *reinterpret_cast<const bf16x8_t*>(&ph[r16 * PS + kq * 8]);
    const bf16x8_t pal = *reinterpret_cast<const bf16x8_t*>(&pl[r16 * PS + kq * 8]);
#pragma unroll
    for (int n = 0; n < NCB; ++n) {
      const bf16x8_t vb = *reinterpret_cast<const bf16x8_t*>(&sVt[(n * 16 + r16) * VS + kq * 8]);
      f32x4_t acc = o[n];
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] *= cr[r];
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pah, vb, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pal, vb, acc, 0, 0, 0);
      o[n] = acc;
    }
  }
  // o[n][r] = O[row 4 kq + r][column 16 n + r16]
  if (nsplit > 1) {
    // partial result of this key range: unnormalised o, with the row's running max and sum
    const int64_t pbase = ((int64_t)blockIdx.x * nsplit + blockIdx.y) * 64;
    if (kq == 0) {
      part_ml[(pbase + myrow) * 2] = m;
      part_ml[(pbase + myrow) * 2 + 1] = l;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = wave * 16 + kq * 4 + r;
#pragma unroll
      for (int n = 0; n < NCB; ++n) {
        const int col = n * 16 + r16;
        if (col < R) part_o[(pbase + row) * R + col] = o[n][r];
      }
    }
    return;
  }
  float inv[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) inv[r] = 1.f / __shfl(l, kq * 4 + r, 64);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = wave * 16 + kq * 4 + r;
    if (row >= ntok * H) continue;
    const int64_t base = ((int64_t)(tok0 + row / H) * H + row % H) * R;
    float w = inv[r];
    if (gate) w *= 1.f / (1.f + expf(-ld(gate + (int64_t)(tok0 + row / H) * gate_stride + row % H)));
#pragma unroll
    for (int n = 0; n < NCB; ++n) {
      const int col = n * 16 + r16;
      if (col < R) st(out + base + col, o[n][r] * w);
    }
  }
}

// Merge the key-range partials of a split step: out = sum_y e^(m_y - M) o_y / sum_y e^(m_y - M) l_y.
__global__ __launch_bounds__(NT) void latent_attention_merge_kernel(const int* __restrict__ items, int nsplit,
                                                                   const float* __restrict__ part_o,
                                                                   const float* __restrict__ part_ml, int H, int R,
                                                                   bf16_t* __restrict__ out,
                                                                   const bf16_t* __restrict__ gate,
                                                                   int64_t gate_stride) {
  const int item = blockIdx.x, row = blockIdx.y;
  const int tok0 = items[item * 3 + 1], ntok = items[item * 3 + 2];
  if (row >= ntok * H) return;
  float M = -INFINITY;
  for (int y = 0; y < nsplit; ++y) M = fmaxf(M, part_ml[(((int64_t)item * nsplit + y) * 64 + row) * 2]);
  float L = 0.f;
  for (int y = 0; y < nsplit; ++y) {
    const float* ml = part_ml + (((int64_t)item * nsplit + y) * 64 + row) * 2;
    L += expf(ml[0] - M) * ml[1];  // an empty range has m = -inf, l = 0
  }
  const int64_t obase = ((int64_t)(tok0 + row / H) * H + row % H) * R;
  if (gate) L *= 1.f + expf(-ld(gate + (int64_t)(tok0 + row / H) * gate_stride + row % H));  // a / L * sigmoid
  for (int c = threadIdx.x; c < R; c += NT) {
    float a = 0.f;
    for (int y = 0; y < nsplit; ++y) {
      const int64_t pb = ((int64_t)item * nsplit + y) * 64 + row;
      a += expf(part_ml[pb * 2] - M) * part_o[pb * R + c];
    }
    st(out + obase + c, a / L);
  }
}

template <typename T, int RC>
int launch_attn(const void* q_abs, const void* cache, const int* tables, int W, int bs, const int* row_seq,
                const int* row_len, float scale, int H, int R, int Dk, int T_rows, int QT, void* out,
                const void* gate, int64_t gate_stride, hipStream_t stream) {
  // key tile: as many of 64 / 32 / 16 rows as fit beside the queries in 128 KB of LDS
  int KT = 64;
  while (KT > 16 && ((size_t)KT * (Dk + 1) + (size_t)QT * 4 * Dk) * 4 > 128 * 1024) KT >>= 1;
  const size_t lds = ((size_t)KT * (Dk + 1) + (size_t)QT * 4 * Dk) * 4;
  if (lds > 160 * 1024) return 1;
  const dim3 grid((T_rows + QT - 1) / QT, (H + 3) / 4);
  auto go = [&](auto kern) {
    if (lds > 64 * 1024) (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, grid, dim3(NT), lds, stream, (const T*)q_abs, (const T*)cache, tables, W, bs, row_seq,
                       row_len, scale, H, R, Dk, KT, T_rows, (T*)out, (const T*)gate, gate_stride);
  };
  if (QT == 4) go(latent_attention_kernel<T, RC, 4>);
  else go(latent_attention_kernel<T, RC, 1>);
  return 0;
}

}  // namespace

extern "C" {

void sm_latent_rope_cache(const void* q, int64_t q_stride, const void* kv, int64_t kv_stride, const void* norm_w,
                          float eps, const int64_t* positions, const float* cos_sin, int H, int dn, int dr,
                          int rot_dims, int R, const int64_t* slots, void* cache, void* q_abs, int interleaved, int T,
                          int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL((latent_rope_cache_kernel<float>), dim3(T), dim3(NT), 0, stream, (const float*)q, q_stride,
                       (const float*)kv, kv_stride, (const float*)norm_w, eps, positions, cos_sin, H, dn, dr,
                       rot_dims, R, slots, (float*)cache, (float*)q_abs, interleaved);
  else
    hipLaunchKernelGGL((latent_rope_cache_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, (const bf16_t*)q, q_stride,
                       (const bf16_t*)kv, kv_stride, (const bf16_t*)norm_w, eps, positions, cos_sin, H, dn, dr,
                       rot_dims, R, slots, (bf16_t*)cache, (bf16_t*)q_abs, interleaved);
}

// Returns 0, or 1 when the sizes do not fit the kernel (R > 1024 or rows too wide for LDS).
int sm_latent_attention(const void* q_abs, const void* cache, const int* tables, int W, int bs, const int* row_seq,
                        const int* row_len, float scale, int H, int R, int Dk, int T, int QT, void* out, int f32,
                        const void* gate, int64_t gate_stride, hipStream_t stream) {
  if (T == 0) return 0;
  const int rc = (R + 63) / 64;
#define SM_GO(TYPE, RC) return launch_attn<TYPE, RC>(q_abs, cache, tables, W, bs, row_seq, row_len, scale, H, R, Dk, T, QT, out, gate, gate_stride, stream)
  if (f32) {
    if (rc <= 1) SM_GO(float, 1);
    if (rc <= 2) SM_GO(float, 2);
    if (rc <= 4) SM_GO(float, 4);
    if (rc <= 8) SM_GO(float, 8);
    if (rc <= 16) SM_GO(float, 16);
  } else {
    if (rc <= 1) SM_GO(bf16_t, 1);
    if (rc <= 2) SM_GO(bf16_t, 2);
    if (rc <= 4) SM_GO(bf16_t, 4);
    if (rc <= 8) SM_GO(bf16_t, 8);
    if (rc <= 16) SM_GO(bf16_t, 16);
  }
#undef SM_GO
  return 1;
}

// bf16, matrix cores. items [n, 3] = (sequence, first token row, tokens), tokens * H <= 64.
// nsplit > 1: every item's keys are cut into nsplit ranges of split_keys (a multiple of 32) that
// run as separate workgroups; part_o [n * nsplit * 64 * R] and part_ml [n * nsplit * 64 * 2] fp32
// hold their partial results and a second kernel merges them.
// Returns 0, or 1 when the sizes are outside the compiled forms (Dk > 576, R > 512, H > 64).
int sm_latent_attention_mfma(const void* q_abs, const void* cache, const int* tables, int W, int bs, const int* items,
                             int n_items, const int* row_len, float scale, int H, int R, int Dk, void* out,
                             int nsplit, int split_keys, float* part_o, float* part_ml, const void* gate,
                             int64_t gate_stride, hipStream_t stream) {
  if (n_items == 0) return 0;
  const int nks = (Dk + 31) / 32, ncb = (R + 15) / 16;
  if (H > 64 || nks > 18 || ncb > 32) return 1;
  const dim3 grid(n_items, nsplit);
#define SM_GO(NKS, NCB)                                                                                            \
  hipLaunchKernelGGL((latent_attention_mfma_kernel<NKS, NCB>), grid, dim3(NT), 0, stream, (const bf16_t*)q_abs,     \
                     (const bf16_t*)cache, tables, W, bs, items, row_len, scale, H, R, Dk, (bf16_t*)out, split_keys, \
                     part_o, part_ml, nsplit > 1 ? nullptr : (const bf16_t*)gate, gate_stride)
  if (nks <= 3 && ncb <= 4) SM_GO(3, 4);
  else if (nks <= 6 && ncb <= 8) SM_GO(6, 8);
  else if (nks <= 10 && ncb <= 16) SM_GO(10, 16);
  else SM_GO(18, 32);
#undef SM_GO
  if (nsplit > 1)
    hipLaunchKernelGGL(latent_attention_merge_kernel, dim3(n_items, 64), dim3(NT), 0, stream, items, nsplit, part_o,
                       part_ml, H, R, (bf16_t*)out, (const bf16_t*)gate, gate_stride);
  return 0;
}

}  // extern "C"
