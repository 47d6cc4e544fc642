// Grouped-query softmax attention with separate key and value sizes over a paged cache. A page of
// one kv head holds bs * (dim + vdim) elements: the keys [bs, dim] row-major, then the values
// TRANSPOSED [vdim, bs] - a value column's keys are contiguous, so both tiles of the matrix-core
// kernel are 16-byte loads and 16-byte LDS writes with nothing to transpose. The cache tensor is
// [blocks, Hkv, bs, dim + vdim] by size only.
//
// qkv_rope_cache: one workgroup per token over the fused projection [q | k | v | ...]: bias add,
//   rotary on the first rot_dims dimensions of every q and k head (pairs (2i, 2i+1) or
//   (i, i + rot_dims/2); angles from an fp32 [cos | sin] table), division of each head by its
//   root mean square, value mixing with an earlier layer's values, query and cache writes. A wave
//   owns a head (its elements in registers); everything is fp32 until the store.
// grouped_attention (fp32 FMA form): workgroup = QT consecutive token rows x up to 4 query heads
//   of ONE kv head (a wave per head). Keys and values stream through LDS in fp32 tiles; a lane
//   scores one key, the wave keeps an online softmax per (row, head), lanes then own value columns.
// grouped_attention_mfma (bf16): a workgroup takes one work item - up to 64 or 128 (token, head of
//   the group) rows of one sequence and kv head, one or two blocks of 16 rows per wave. Key tiles of
//   32 in LDS (keys row-major, values transposed as in the cache), S^T = K Q^T and O += P V on
//   v_mfma_f32_16x16x32_bf16; fp32 online softmax in base 2; P enters the second product as a bf16
//   pair (hi + lo) straight from the registers the scores arrive in. Decode-only steps cut the keys into ranges over blockIdx.z and a merge kernel
//   joins them.
// Both forms multiply the result by sigmoid(gate) when a gate is given. A row's result depends
// only on its own keys and the fixed tile sizes.
// Score options of both forms (each may be off): slopes [Hq] - the score of query i and key j loses
// slopes[h] (i - j); chunk - query i sees only keys j >= (i / chunk) chunk; sinks [Hq] - one more
// score per head that enters the softmax's denominator and has no value (the running maximum and
// sum start from it instead of from nothing). Key tiles start at multiples of the tile size from
// position 0, so a row's tiles do not depend on what else the step holds.
// window / keep: query i sees key j <= i only if i - j < window or j < keep (the sequence's first
// tokens stay visible); the tiles between the kept tokens and the first window of a work item are
// skipped. qkv_rope_cache options: norm_first - the unit norm and its weights come before the
// rotation; v_from_k - the values are the biased key projections themselves (no value columns).
#include "seqmix_common.h"
#include <algorithm>

using namespace sm;

namespace {

constexpr int NT = 256;
constexpr int MAXE = 8;  // head elements per lane: dim <= 512

template <typename T>
__global__ __launch_bounds__(NT) void qkv_rope_cache_kernel(
    const T* __restrict__ qkv, int64_t stride, const float* __restrict__ bias, const int64_t* __restrict__ positions,
    const float* __restrict__ cos_sin, int Hq, int Hkv, int dim, int vdim, int rot_dims, int interleaved, int unit,
    float eps, float* __restrict__ v_first, int v_mode, float lam, const int64_t* __restrict__ slots,
    T* __restrict__ cache, int bs, T* __restrict__ q_out, const float* __restrict__ qk_w, int norm_first,
    int v_from_k) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int half = rot_dims >> 1;
  const float* cs = rot_dims ? cos_sin + positions[t] * rot_dims : nullptr;  // [cos(half) | sin(half)]
  const T* row = qkv + t * stride;
  const int64_t slot = slots[t];
  const int Dr = dim + vdim;
  const int64_t blk = slot >= 0 ? slot / bs : 0, off = slot >= 0 ? slot % bs : 0;
  // blockIdx.y spreads a token's heads (a wave each) and value elements over workgroups: a step of
  // few tokens still fills the chip
  for (int hd = blockIdx.y * (NT / 64) + wave; hd < Hq + Hkv; hd += gridDim.y * (NT / 64)) {
    const bool is_q = hd < Hq;
    const int col0 = is_q ? hd * dim : Hq * dim + (hd - Hq) * dim;
    const float* nw = qk_w ? qk_w + (is_q ? 0 : dim) : nullptr;  // the norm's weight, shared by the heads
    const float* nw1 = norm_first ? nw : nullptr;               // applied before the rotation
    float r[MAXE];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAXE; ++i) {
      const int e = lane + 64 * i;
      float v = 0.f, raw = 0.f;
      if (e < dim) {
        raw = ld(row + col0 + e) + (bias ? bias[col0 + e] : 0.f);
        const float x = nw1 ? raw * nw1[e] : raw;
        v = x;
        if (e < rot_dims) {
          int p, f;
          bool first;
          if (interleaved) {
            p = e ^ 1;
            f = e >> 1;
            first = (e & 1) == 0;
          } else {
            first = e < half;
            p = first ? e + half : e - half;
            f = first ? e : e - half;
          }
          const float xp = (ld(row + col0 + p) + (bias ? bias[col0 + p] : 0.f)) * (nw1 ? nw1[p] : 1.f);
          const float c = cs[f], s = cs[half + f];
          v = first ? x * c - xp * s : x * c + xp * s;
        }
      }
      r[i] = v;
      ss += norm_first ? raw * raw : v * v;
    }
    float inv = 1.f;
    if (unit) inv = 1.f / sqrtf(wave_sum(ss) / (float)dim + eps);
    T* dst = nullptr;
    if (is_q) dst = q_out + (t * Hq + hd) * dim;
    else if (slot >= 0) dst = cache + (blk * Hkv + (hd - Hq)) * bs * Dr + off * dim;
    if (dst == nullptr) continue;
#pragma unroll
    for (int i = 0; i < MAXE; ++i) {
      const int e = lane + 64 * i;
      if (e < dim) st(dst + e, r[i] * inv * ((nw && !norm_first) ? nw[e] : 1.f));
    }
  }
  const int nv = Hkv * vdim, vcol0 = v_from_k ? Hq * dim : (Hq + Hkv) * dim;
  for (int e = blockIdx.y * NT + threadIdx.x; e < nv; e += gridDim.y * NT) {
    float v = ld(row + vcol0 + e) + (bias ? bias[vcol0 + e] : 0.f);
    if (v_mode == 1) v_first[t * nv + e] = v;
    else if (v_mode == 2) v = (1.f - lam) * v + lam * v_first[t * nv + e];
    if (slot >= 0) {
      const int g = e / vdim, c = e - g * vdim;
      st(cache + (blk * Hkv + g) * bs * Dr + (int64_t)bs * dim + (int64_t)c * bs + off, v);  // transposed
    }
  }
}

// bf16 form with 16-byte accesses: a head is dim / 8 lanes, each with eight consecutive elements (four
// interleaved pairs, or one eighth of a half with its partner chunk loaded beside it). Needs
// dim = 8 * 2^k <= 512, rotary dims a multiple of 8 (16 for the half-split pairing) and 16-byte
// aligned rows; the launcher falls back to the element-wise kernel otherwise.
__device__ __forceinline__ void ld8(const bf16_t* p, float (&v)[8]) {
  const uint4 t = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ void add8(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w;
  v[4] += b.x; v[5] += b.y; v[6] += b.z; v[7] += b.w;
}
__device__ __forceinline__ void st8(bf16_t* p, const float (&v)[8], float mul) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const __bf16 a = (__bf16)(v[2 * i] * mul), b = (__bf16)(v[2 * i + 1] * mul);  // round to nearest even
    w[i] = (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
  }
  *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
}

__global__ __launch_bounds__(NT) void qkv_rope_cache_vec_kernel(
    const bf16_t* __restrict__ qkv, int64_t stride, const float* __restrict__ bias,
    const int64_t* __restrict__ positions, const float* __restrict__ cos_sin, int Hq, int Hkv, int dim, int vdim,
    int rot_dims, int interleaved, int unit, float eps, float* __restrict__ v_first, int v_mode, float lam,
    const int64_t* __restrict__ slots, bf16_t* __restrict__ cache, int bs, bf16_t* __restrict__ q_out,
    const float* __restrict__ qk_w, int norm_first, int v_from_k) {
  const int64_t t = blockIdx.x;
  const int half = rot_dims >> 1;
  const float* cs = rot_dims ? cos_sin + positions[t] * rot_dims : nullptr;  // [cos(half) | sin(half)]
  const bf16_t* row = qkv + t * stride;
  const int64_t slot = slots[t];
  const int Dr = dim + vdim;
  const int64_t blk = slot >= 0 ? slot / bs : 0, off = slot >= 0 ? slot % bs : 0;
  const int lph = dim >> 3, hpp = NT / lph;  // lanes per head, heads per pass
  const int c = threadIdx.x & (lph - 1), hl = threadIdx.x / lph;
  for (int h0 = blockIdx.y * hpp; h0 < Hq + Hkv; h0 += gridDim.y * hpp) {
    const int hd = h0 + hl;
    const bool on = hd < Hq + Hkv;
    const int col = hd * dim + c * 8;  // q heads, then k heads, back to back in the projection
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float ss = 0.f;
    const float* nw = qk_w ? qk_w + (hd < Hq ? 0 : dim) : nullptr;
    const float* nw1 = norm_first ? nw : nullptr;  // weights applied before the rotation
    if (on) {
      ld8(row + col, x);
      if (bias) add8(bias + col, x);
      if (norm_first) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          ss += x[i] * x[i];
          if (nw1) x[i] *= nw1[c * 8 + i];
        }
      }
      if (c * 8 < rot_dims) {
        if (interleaved) {
          const float4 co = *reinterpret_cast<const float4*>(cs + c * 4);
          const float4 si = *reinterpret_cast<const float4*>(cs + half + c * 4);
          const float cc[4] = {co.x, co.y, co.z, co.w}, sn[4] = {si.x, si.y, si.z, si.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float u = x[2 * i], v = x[2 * i + 1];
            x[2 * i] = u * cc[i] - v * sn[i];
            x[2 * i + 1] = v * cc[i] + u * sn[i];
          }
        } else {
          const bool first = c * 8 < half;
          const int pc = first ? col + half : col - half;  // the partner chunk
          const int f = first ? c * 8 : c * 8 - half;
          float xp[8], cc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, sn[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          ld8(row + pc, xp);
          if (bias) add8(bias + pc, xp);
          if (nw1) {
#pragma unroll
            for (int i = 0; i < 8; ++i) xp[i] *= nw1[c * 8 + (first ? half : -half) + i];
          }
          add8(cs + f, cc);
          add8(cs + half + f, sn);
#pragma unroll
          for (int i = 0; i < 8; ++i) x[i] = first ? x[i] * cc[i] - xp[i] * sn[i] : x[i] * cc[i] + xp[i] * sn[i];
        }
      }
    }
    float inv = 1.f;
    if (unit) {
      if (!norm_first) {
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
      }
      for (int o = lph >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);  // the head's lanes are an aligned group
      inv = 1.f / sqrtf(ss / (float)dim + eps);
    }
    if (!on) continue;
    if (nw && !norm_first) {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] *= nw[c * 8 + i];
    }
    if (hd < Hq) st8(q_out + (t * Hq + hd) * dim + c * 8, x, inv);
    else if (slot >= 0) st8(cache + (blk * Hkv + (hd - Hq)) * bs * Dr + off * dim + c * 8, x, inv);
  }
  const int nv = Hkv * vdim, vcol0 = v_from_k ? Hq * dim : (Hq + Hkv) * dim;
  for (int e = blockIdx.y * NT + threadIdx.x; e < nv; e += gridDim.y * NT) {
    float v = ld(row + vcol0 + e) + (bias ? bias[vcol0 + e] : 0.f);
    if (v_mode == 1) v_first[t * nv + e] = v;
    else if (v_mode == 2) v = (1.f - lam) * v + lam * v_first[t * nv + e];
    if (slot >= 0) {
      const int g = e / vdim, cc = e - g * vdim;
      st(cache + (blk * Hkv + g) * bs * Dr + (int64_t)bs * dim + (int64_t)cc * bs + off, v);  // transposed
    }
  }
}

// VC = ceil(vdim / 64) output columns per lane; QT token rows per workgroup.
template <typename T, int VC, int QT>
__global__ __launch_bounds__(NT) void grouped_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ cache, const int* __restrict__ tables, int W, int bs,
    const int* __restrict__ row_seq, const int* __restrict__ row_len, float scale, int Hq, int Hkv, int dim, int vdim,
    int KT, int T_rows, const T* __restrict__ gate, int64_t gate_stride, T* __restrict__ out,
    const float* __restrict__ slopes, int chunk, const float* __restrict__ sinks, int window, int keep) {
  extern __shared__ float lds[];
  const int Dr = dim + vdim;
  const int KS = Dr + 1;                 // tile row stride (odd: lanes hit distinct banks)
  float* sK = lds;                       // [KT][KS]  key | value
  float* sQ = lds + KT * KS;             // [QT][4][dim], pre-scaled
  const int G = Hq / Hkv, subs = (G + 3) / 4;
  const int g = blockIdx.y / subs, sub = blockIdx.y - g * subs;
  const int t0 = blockIdx.x * QT;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int hg = sub * 4 + wave;         // head within the group
  const bool head_ok = hg < G;
  const int h = g * G + hg;

  for (int e = threadIdx.x; e < QT * 4 * dim; e += NT) {
    const int r = e / (4 * dim), rem = e - r * 4 * dim;
    const int w = rem / dim, d = rem - w * dim;
    const int t = t0 + r, hh = sub * 4 + w;
    sQ[e] = (t < T_rows && hh < G) ? ld(q + ((int64_t)t * Hq + g * G + hh) * dim + d) * scale : 0.f;
  }

  int seq_r[QT], len_r[QT], lo_r[QT], wlo_r[QT];
  bool done[QT];
  if (window <= 0) keep = 0;
#pragma unroll
  for (int r = 0; r < QT; ++r) {
    const int t = t0 + r;
    done[r] = t >= T_rows;
    seq_r[r] = done[r] ? -1 : row_seq[t];
    len_r[r] = done[r] ? 0 : row_len[t];
    lo_r[r] = (chunk > 0 && len_r[r] > 0) ? ((len_r[r] - 1) / chunk) * chunk : 0;  // first key of the row's chunk
    wlo_r[r] = window > 0 ? max(0, len_r[r] - window) : 0;                          // first key of the row's window
  }
  const float slope = (slopes != nullptr && head_ok) ? slopes[h] : 0.f;
  const bool has_sink = sinks != nullptr && head_ok;
  const float sink = has_sink ? sinks[h] : 0.f;

  for (int pass = 0; pass < QT; ++pass) {
    int seq = -1;
#pragma unroll
    for (int r = 0; r < QT; ++r)
      if (seq < 0 && !done[r]) seq = seq_r[r];
    if (seq < 0) break;
    bool act[QT];
    int maxlen = 0, minlo = 0x7fffffff, minwlo = 0x7fffffff;
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      act[r] = !done[r] && seq_r[r] == seq;
      if (act[r]) {
        maxlen = max(maxlen, len_r[r]);
        minlo = min(minlo, lo_r[r]);
        minwlo = min(minwlo, wlo_r[r]);
      }
    }
    float m[QT], l[QT], acc[QT][VC];
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      m[r] = has_sink ? sink : -INFINITY;  // the sink is a score that is already counted
      l[r] = has_sink ? 1.f : 0.f;
#pragma unroll
      for (int c = 0; c < VC; ++c) acc[r][c] = 0.f;
    }
    const int* bt = tables + (int64_t)seq * W;
    bool first_tile = true;
    for (int k0 = (minlo / KT) * KT; k0 < maxlen; k0 += KT) {
      // a tile past the kept first tokens and before every row's window holds nothing visible
      if (!first_tile && k0 >= keep && k0 + KT <= minwlo) continue;
      first_tile = false;  // the first pass always runs: its barrier orders the query tile's writes
      __syncthreads();  // previous tile fully used (and sQ written, first time)
      for (int e = threadIdx.x; e < KT * dim; e += NT) {  // keys: row-major in the page
        const int j = e / dim, d = e - j * dim;
        const int key = k0 + j;
        float v = 0.f;
        if (key < maxlen) v = ld(cache + ((int64_t)bt[key / bs] * Hkv + g) * bs * Dr + (int64_t)(key % bs) * dim + d);
        sK[j * KS + d] = v;
      }
      for (int e = threadIdx.x; e < KT * vdim; e += NT) {  // values: transposed in the page, lanes along keys
        const int d = e / KT, j = e - d * KT;
        const int key = k0 + j;
        float v = 0.f;
        if (key < maxlen)
          v = ld(cache + ((int64_t)bt[key / bs] * Hkv + g) * bs * Dr + (int64_t)bs * dim + (int64_t)d * bs + (key % bs));
        sK[j * KS + dim + d] = v;
      }
      __syncthreads();
      if (!head_ok) continue;
#pragma unroll
      for (int r = 0; r < QT; ++r) {
        if (!act[r] || k0 >= len_r[r] || k0 + KT <= lo_r[r] || (k0 >= keep && k0 + KT <= wlo_r[r])) continue;
        const bool valid = lane < KT && k0 + lane < len_r[r] && k0 + lane >= lo_r[r] &&
                           (k0 + lane >= wlo_r[r] || k0 + lane < keep);
        float s = -INFINITY;
        if (valid) {
          const float* qv = sQ + (r * 4 + wave) * dim;
          const float* kr = sK + lane * KS;
          float a = 0.f;
          for (int d = 0; d < dim; ++d) a += qv[d] * kr[d];
          s = a - slope * (float)(len_r[r] - 1 - (k0 + lane));
        }
        const float mn = fmaxf(m[r], wave_max(s));
        const float corr = expf(m[r] - mn);  // exp(-inf) = 0 on the first tile
        const float p = valid ? expf(s - mn) : 0.f;
        l[r] = l[r] * corr + wave_sum(p);
        m[r] = mn;
#pragma unroll
        for (int c = 0; c < VC; ++c) acc[r][c] *= corr;
        const int nk = min(KT, len_r[r] - k0);
        for (int j = max(0, lo_r[r] - k0); j < nk; ++j) {
          const float pj = __shfl(p, j, 64);
          const float* vr = sK + j * KS + dim;
#pragma unroll
          for (int c = 0; c < VC; ++c) {
            const int col = lane + 64 * c;
            if (col < vdim) acc[r][c] += pj * vr[col];
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      if (!act[r]) continue;
      done[r] = true;
      if (!head_ok) continue;
      const float inv = 1.f / l[r];
#pragma unroll
      for (int c = 0; c < VC; ++c) {
        const int col = lane + 64 * c;
        if (col >= vdim) continue;
        float o = acc[r][c] * inv;
        if (gate) o *= 1.f / (1.f + expf(-ld(gate + (int64_t)(t0 + r) * gate_stride + h * vdim + col)));
        st(out + ((int64_t)(t0 + r) * Hq + h) * vdim + col, o);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int MKT = 32;  // keys per tile

// DkP = 32 NKS >= dim and VP = 16 NCB >= vdim are the padded sizes (zeros in LDS and in the
// query fragments). items [n, 3] = (sequence, first token row, tokens), tokens * G <= 64 RB: a wave
// owns RB blocks of 16 rows (block rb of wave w = item rows 16 (4 rb + w) ..), so a key tile's
// fragments are read from LDS once for RB row blocks. The next tile's global loads are issued
// before the current tile's products, so their latency runs beside the matrix work.
template <int NKS, int NCB, int RB>
__global__ __launch_bounds__(NT) void grouped_attention_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache, const int* __restrict__ tables, int W, int bs,
    const int* __restrict__ items, const int* __restrict__ row_len, float scale, int Hq, int Hkv, int dim, int vdim,
    const bf16_t* __restrict__ gate, int64_t gate_stride, bf16_t* __restrict__ out, int split_keys,
    float* __restrict__ part_o, float* __restrict__ part_ml, const float* __restrict__ slopes, int chunk,
    const float* __restrict__ sinks, int window, int keep) {
  constexpr int DkP = 32 * NKS, VP = 16 * NCB;
  constexpr int KS = DkP + 8, VS = MKT + 8;  // LDS row strides (bf16), 16-byte multiples
  // Two tile buffers for the small forms: the next tile is written while the current one is read and
  // one barrier per tile is enough. The 256 / 256 form keeps one buffer (two would leave one
  // workgroup per CU) and brackets the write with two barriers.
  constexpr int NBUF = NKS <= 4 ? 2 : 1;
  __shared__ __attribute__((aligned(16))) bf16_t sK[NBUF * MKT * KS];
  __shared__ __attribute__((aligned(16))) bf16_t sVt[NBUF * VP * VS];
  // the kv head is the fastest grid index: the workgroups of one item follow each other
  const int item = blockIdx.y, g = blockIdx.x, G = Hq / Hkv, Dr = dim + vdim;
  const int seq = items[item * 3], tok0 = items[item * 3 + 1], ntok = items[item * 3 + 2];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, kq = lane >> 4;
  // this lane's query rows (as the B operand's column): item row 16 (4 rb + wave) + r16
  int mytok[RB], myhead[RB], mylen[RB], mylo[RB], mywlo[RB];
  float myslope[RB];  // in base 2, like the scores
  if (window <= 0) keep = 0;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int myrow = (rb * 4 + wave) * 16 + r16;
    const bool ok = myrow < ntok * G;
    mytok[rb] = tok0 + (ok ? myrow / G : 0);
    myhead[rb] = g * G + (ok ? myrow % G : 0);
    mylen[rb] = ok ? row_len[mytok[rb]] : 0;
    mylo[rb] = (chunk > 0 && mylen[rb] > 0) ? ((mylen[rb] - 1) / chunk) * chunk : 0;  // first key of the row's chunk
    mywlo[rb] = window > 0 ? max(0, mylen[rb] - window) : 0;                             // first key of the row's window
    myslope[rb] = slopes ? slopes[myhead[rb]] * 1.44269504088896341f : 0.f;
  }
  const int maxlen = row_len[tok0 + ntok - 1];  // the run's last token sees the most keys
  // the run's first token starts the earliest chunk; tiles start at multiples of 32 from position 0
  const int kbase = chunk > 0 ? ((((row_len[tok0] - 1) / chunk) * chunk) / MKT) * MKT : 0;
  // A window leaves a gap between the tiles of the kept first tokens [0, keepT) and the tile that the
  // run's first window starts in. The tile loop runs over positions v with the gap taken out:
  // key = v below keepT, v + gap from there on; the decode split cuts [0, vlen) too.
  int keepT = 0, gap = 0;
  if (window > 0) {
    keepT = ((keep + MKT - 1) / MKT) * MKT;
    const int wbase = (max(0, row_len[tok0] - window) / MKT) * MKT;
    gap = max(0, wbase - keepT);
  }
  const int vlen = maxlen - gap;
  auto key_of = [&](int v) { return v + (v >= keepT ? gap : 0); };

  // padding columns of the key tile and padding rows of the value tile stay zero for the whole kernel
  for (int e = threadIdx.x; e < NBUF * MKT * KS; e += NT) sK[e] = 0;
  for (int e = threadIdx.x; e < NBUF * VP * VS; e += NT) sVt[e] = 0;

  bf16x8_t qf[RB][NKS];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int d = ks * 32 + kq * 8 + i;
        const bf16_t w = (mylen[rb] > 0 && d < dim) ? q[((int64_t)mytok[rb] * Hq + myhead[rb]) * dim + d] : (bf16_t)0;
        qf[rb][ks][i] = __builtin_bit_cast(__bf16, w);
      }
    }
  f32x4_t o[RB][NCB];
  float m[RB], l[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    // a sink is a score that is already counted (by the first key range only)
    const bool sk = sinks != nullptr && blockIdx.z == 0;
    m[rb] = sk ? sinks[myhead[rb]] * 1.44269504088896341f : -INFINITY;
    l[rb] = sk ? 1.f : 0.f;
#pragma unroll
    for (int n = 0; n < NCB; ++n) o[rb][n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  const int* bt = tables + (int64_t)seq * W;
  const bool vec = (dim & 7) == 0;  // key rows are 16-byte multiples (value columns always: bs % 8 == 0)
  // the softmax runs in base 2 (scores carry log2 e): the hardware exponential is exp2, about one
  // fp32 ulp, far below the bf16 rounding of what the weights multiply
  const float scale2 = scale * 1.44269504088896341f;

  // decode steps split a row's keys over blockIdx.z: this workgroup takes [kbeg, kend)
  const int nsplit = gridDim.z;
  // (ranges are whole tiles, so a tile's keys need only stay below maxlen)
  const int kbeg = nsplit > 1 ? kbase + blockIdx.z * split_keys : kbase;
  const int kend = nsplit > 1 ? min(vlen, kbeg + split_keys) : vlen;
  constexpr int CK = DkP / 8;                      // 16-byte chunks per key row (padded)
  constexpr int NCK = (MKT * CK + NT - 1) / NT;    // key chunks per thread
  constexpr int CV = MKT / 8;                      // chunks per value column (8 keys each)
  constexpr int NCV = (VP * CV + NT - 1) / NT;     // value chunks per thread
  const bool one_page = (bs % MKT) == 0;           // a tile lies inside one page (tiles start at multiples of 32)
  // All of a tile's 16-byte chunks are requested before any is used: key rows with lanes along the
  // row, value columns with lanes along the keys - both contiguous in the page. Keys at or beyond
  // kend are zeroed (a page's unwritten rest may hold anything, and 0 x NaN would spoil a column).
  u32x4_t pk[NCK], pv[NCV];
  // one-page tiles: the tile's page and its first row in the page advance without a division
  int tile_page = 0, tile_off = 0, tile_next = -1;
  auto fetch = [&](int k0) {
    if (one_page && k0 != tile_next) {  // the first tile, and the one after the gap
      tile_page = k0 / bs;
      tile_off = k0 % bs;
    }
    tile_next = k0 + MKT;
    const int64_t page0 = one_page ? ((int64_t)bt[tile_page] * Hkv + g) * bs * Dr : 0;
    const int off0 = tile_off;
    if (one_page) {
      tile_off += MKT;
      if (tile_off >= bs) {
        tile_off = 0;
        ++tile_page;
      }
    }
#pragma unroll
    for (int i = 0; i < NCK; ++i) {
      const int e = threadIdx.x + i * NT;
      const int j = e / CK, c = e - j * CK;
      const int key = k0 + j;
      u32x4_t v = {0, 0, 0, 0};
      if (e < MKT * CK && c * 8 < dim && key < maxlen) {
        const int64_t page = one_page ? page0 : ((int64_t)bt[key / bs] * Hkv + g) * bs * Dr;
        const int off = one_page ? off0 + j : key % bs;
        const bf16_t* src = cache + page + (int64_t)off * dim + c * 8;
        if (vec) {
          v = *reinterpret_cast<const u32x4_t*>(src);
        } else {
#pragma unroll
          for (int qq = 0; qq < 8; ++qq)
            if (c * 8 + qq < dim) v[qq >> 1] |= (uint32_t)src[qq] << (16 * (qq & 1));
        }
      }
      pk[i] = v;
    }
#pragma unroll
    for (int i = 0; i < NCV; ++i) {
      const int e = threadIdx.x + i * NT;
      const int d = e / CV, j8 = e - d * CV;
      const int key = k0 + j8 * 8;
      u32x4_t v = {0, 0, 0, 0};
      if (d < vdim && key < maxlen) {
        const int64_t page = one_page ? page0 : ((int64_t)bt[key / bs] * Hkv + g) * bs * Dr;
        const int off = one_page ? off0 + j8 * 8 : key % bs;
        v = *reinterpret_cast<const u32x4_t*>(cache + page + (int64_t)bs * dim + (int64_t)d * bs + off);
        const int nv = maxlen - key;  // keys of this chunk that exist
        if (nv < 8) {
#pragma unroll
          for (int w = 0; w < 4; ++w) v[w] = 2 * w + 1 < nv ? v[w] : (2 * w < nv ? v[w] & 0xffffu : 0u);
        }
      }
      pv[i] = v;
    }
  };
  auto stage = [&](int buf) {  // the fetched tile -> LDS buffer buf
    bf16_t* const kb_ = sK + buf * MKT * KS;
    bf16_t* const vb_ = sVt + buf * VP * VS;
#pragma unroll
    for (int i = 0; i < NCK; ++i) {
      const int e = threadIdx.x + i * NT;
      const int j = e / CK, c = e - j * CK;
      if (e < MKT * CK && c * 8 < dim) *reinterpret_cast<u32x4_t*>(&kb_[j * KS + c * 8]) = pk[i];
    }
#pragma unroll
    for (int i = 0; i < NCV; ++i) {
      const int e = threadIdx.x + i * NT;
      const int d = e / CV, j8 = e - d * CV;
      // a value column's keys are stored in the order the weights arrive in: position 8 q + i holds
      // key 4 q + i (i < 4) or key 16 + 4 q + i - 4, so one 16-byte read gives a lane its eight keys
      if (d < vdim) {
        const int base = d * VS + (j8 & 1) * 16 + (j8 >> 1) * 4;
        *reinterpret_cast<uint2*>(&vb_[base]) = make_uint2(pv[i][0], pv[i][1]);
        *reinterpret_cast<uint2*>(&vb_[base + 8]) = make_uint2(pv[i][2], pv[i][3]);
      }
    }
  };
  if (kbeg < kend) fetch(key_of(kbeg));
  if (NBUF == 2) {
    __syncthreads();  // the zero fill is done
    stage(0);
    if (kbeg + MKT < kend) fetch(key_of(kbeg + MKT));
    __syncthreads();
  }
  int it = 0;
  for (int v0 = kbeg; v0 < kend; v0 += MKT, ++it) {
    const int k0 = key_of(v0);
    const int cur = NBUF == 2 ? (it & 1) : 0;
    if (NBUF == 1) {
      __syncthreads();  // the previous tile is no longer read (first time: the zero fill is done)
      stage(0);
      __syncthreads();
      if (v0 + MKT < kend) fetch(key_of(v0 + MKT));  // in flight during this tile's products
    }
    const bf16_t* const tK = sK + cur * MKT * KS;
    const bf16_t* const tV = sVt + cur * VP * VS;
    // scores of this lane's rows against keys k0 + 16 kb + 4 kq + r
    float sc[RB][2][4];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      f32x4_t a[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) a[rb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const bf16x8_t ka = *reinterpret_cast<const bf16x8_t*>(&tK[(kb * 16 + r16) * KS + ks * 32 + kq * 8]);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) a[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[rb][ks], a[rb], 0, 0, 0);
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = k0 + kb * 16 + kq * 4 + r;
          sc[rb][kb][r] = (key < mylen[rb] && key >= mylo[rb] && (key >= mywlo[rb] || key < keep))
                              ? a[rb][r] * scale2 - myslope[rb] * (float)(mylen[rb] - 1 - key)
                              : -INFINITY;
        }
    }
    // The weights never pass through LDS. After S^T = K Q^T this lane holds, for its query row r16,
    // the keys 4 kq .. 4 kq + 3 of both 16-key halves of the tile - eight keys, which is exactly one
    // A operand of the second product if the contraction index is ordered that way; the value
    // operand below is read in the same order (the order of a contraction is free as long as both
    // operands agree).
    float cr[RB][4];
    bool rescale[RB];  // wave-uniform: some row's maximum moved in this tile
    bf16x8_t pah[RB], pal[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) mx = fmaxf(mx, sc[rb][kb][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float mn = fmaxf(m[rb], mx);
      const float mref = (mn == -INFINITY) ? 0.f : mn;  // a row with no key yet
      const float corr = __builtin_amdgcn_exp2f(m[rb] - mref);
      float psum = 0.f;
      u32x4_t hw, lw;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        // hi = the weight's upper 16 bits (truncated), lo = the upper 16 bits of the exact rest:
        // hi + lo differs from the fp32 weight by less than 2^-16 of it, with no rounding arithmetic.
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          const float p0 = __builtin_amdgcn_exp2f(sc[rb][kb][r] - mref);
          const float p1 = __builtin_amdgcn_exp2f(sc[rb][kb][r + 1] - mref);
          psum += p0 + p1;
          const uint32_t u0 = __float_as_uint(p0), u1 = __float_as_uint(p1);
          const uint32_t h0 = u0 & 0xffff0000u, h1 = u1 & 0xffff0000u;
          const uint32_t r0 = __float_as_uint(p0 - __uint_as_float(h0)), r1 = __float_as_uint(p1 - __uint_as_float(h1));
          hw[kb * 2 + (r >> 1)] = (h0 >> 16) | h1;
          lw[kb * 2 + (r >> 1)] = (r0 >> 16) | (r1 & 0xffff0000u);
        }
      }
      pah[rb] = __builtin_bit_cast(bf16x8_t, hw);
      pal[rb] = __builtin_bit_cast(bf16x8_t, lw);
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      l[rb] = l[rb] * corr + psum;
      m[rb] = mn;
      // the accumulators hold rows 4 kq + r: their correction comes from the lane that owns the row
#pragma unroll
      for (int r = 0; r < 4; ++r) cr[rb][r] = __shfl(corr, kq * 4 + r, 64);
      rescale[rb] = __any(corr != 1.f);
    }
#pragma unroll
    for (int n = 0; n < NCB; ++n) {
      const bf16x8_t vb = *reinterpret_cast<const bf16x8_t*>(&tV[(n * 16 + r16) * VS + kq * 8]);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        f32x4_t acc = o[rb][n];
        if (rescale[rb]) {
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[r] *= cr[rb][r];
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pah[rb], vb, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pal[rb], vb, acc, 0, 0, 0);
        o[rb][n] = acc;
      }
    }
    if (NBUF == 2) {
      // every wave has finished the previous tile (barrier below, one iteration ago), so the other
      // buffer is free: write the next tile there and ask for the one after it
      if (v0 + MKT < kend) {
        stage(cur ^ 1);
        if (v0 + 2 * MKT < kend) fetch(key_of(v0 + 2 * MKT));
      }
      __syncthreads();
    }
  }
  // o[rb][n][r] = O[row 16 (4 rb + wave) + 4 kq + r][column 16 n + r16]
  if (nsplit > 1) {  // RB == 1 (the host splits decode-only steps, whose items have at most 64 rows)
    const int64_t pbase = (((int64_t)item * Hkv + g) * nsplit + blockIdx.z) * 64;
    if (kq == 0) {
      part_ml[(pbase + wave * 16 + r16) * 2] = m[0];
      part_ml[(pbase + wave * 16 + r16) * 2 + 1] = l[0];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = wave * 16 + kq * 4 + r;
#pragma unroll
      for (int n = 0; n < NCB; ++n) {
        const int col = n * 16 + r16;
        if (col < vdim) part_o[(pbase + row) * vdim + col] = o[0][n][r];
      }
    }
    return;
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float inv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) inv[r] = 1.f / __shfl(l[rb], kq * 4 + r, 64);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = (rb * 4 + wave) * 16 + kq * 4 + r;
      if (row >= ntok * G) continue;
      const int64_t tok = tok0 + row / G;
      const int h = g * G + row % G;
#pragma unroll
      for (int n = 0; n < NCB; ++n) {
        const int col = n * 16 + r16;
        if (col >= vdim) continue;
        float v = o[rb][n][r] * inv[r];
        if (gate) v *= 1.f / (1.f + expf(-ld(gate + tok * gate_stride + h * vdim + col)));
        st(out + (tok * Hq + h) * vdim + col, v);
      }
    }
  }
}

// Merge the key-range partials of a split step: out = sum_z 2^(m_z - M) o_z / sum_z 2^(m_z - M) l_z.
__global__ __launch_bounds__(NT) void grouped_attention_merge_kernel(
    const int* __restrict__ items, int nsplit, const float* __restrict__ part_o, const float* __restrict__ part_ml,
    int Hq, int Hkv, int vdim, const bf16_t* __restrict__ gate, int64_t gate_stride, bf16_t* __restrict__ out) {
  const int item = blockIdx.x, g = blockIdx.y, row = blockIdx.z;
  const int G = Hq / Hkv;
  const int tok0 = items[item * 3 + 1], ntok = items[item * 3 + 2];
  if (row >= ntok * G) return;
  const int64_t base = ((int64_t)item * Hkv + g) * nsplit;
  float M = -INFINITY;
  for (int z = 0; z < nsplit; ++z) M = fmaxf(M, part_ml[((base + z) * 64 + row) * 2]);
  float L = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float* ml = part_ml + ((base + z) * 64 + row) * 2;
    L += exp2f(ml[0] - M) * ml[1];  // maxima are in base 2; an empty range has m = -inf, l = 0
  }
  const int64_t tok = tok0 + row / G;
  const int h = g * G + row % G;
  for (int c = threadIdx.x; c < vdim; c += NT) {
    float a = 0.f;
    for (int z = 0; z < nsplit; ++z) {
      const int64_t pb = (base + z) * 64 + row;
      a += exp2f(part_ml[pb * 2] - M) * part_o[pb * vdim + c];
    }
    float v = a / L;
    if (gate) v *= 1.f / (1.f + expf(-ld(gate + tok * gate_stride + h * vdim + c)));
    st(out + (tok * Hq + h) * vdim + c, v);
  }
}

template <typename T, int VC>
int launch_attn(const void* q, const void* cache, const int* tables, int W, int bs, const int* row_seq,
                const int* row_len, float scale, int Hq, int Hkv, int dim, int vdim, int T_rows, int QT,
                const void* gate, int64_t gate_stride, void* out, const float* slopes, int chunk, const float* sinks,
                int window, int keep, hipStream_t stream) {
  const int Dr = dim + vdim;
  int KT = 64;
  while (KT > 16 && ((size_t)KT * (Dr + 1) + (size_t)QT * 4 * dim) * 4 > 128 * 1024) KT >>= 1;
  const size_t lds = ((size_t)KT * (Dr + 1) + (size_t)QT * 4 * dim) * 4;
  if (lds > 160 * 1024) return 1;
  const int G = Hq / Hkv;
  const dim3 grid((T_rows + QT - 1) / QT, Hkv * ((G + 3) / 4));
  auto go = [&](auto kern) {
    if (lds > 64 * 1024) (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, grid, dim3(NT), lds, stream, (const T*)q, (const T*)cache, tables, W, bs, row_seq, row_len,
                       scale, Hq, Hkv, dim, vdim, KT, T_rows, (const T*)gate, gate_stride, (T*)out, slopes, chunk, sinks,
                       window, keep);
  };
  if (QT == 4) go(grouped_attention_kernel<T, VC, 4>);
  else go(grouped_attention_kernel<T, VC, 1>);
  return 0;
}

}  // namespace

extern "C" {

void sm_qkv_rope_cache(const void* qkv, int64_t stride, const float* bias, const int64_t* positions,
                       const float* cos_sin, int Hq, int Hkv, int dim, int vdim, int rot_dims, int interleaved,
                       int unit, float eps, float* v_first, int v_mode, float lam, const int64_t* slots, void* cache,
                       int bs, void* q_out, const float* qk_w, int norm_first, int v_from_k, int T, int f32,
                       hipStream_t stream) {
  if (T == 0) return;
  // workgroups per token: all heads in parallel for small steps, fewer as the step grows
  const int per_tok = (Hq + Hkv + NT / 64 - 1) / (NT / 64);
  const int gy = std::max(1, std::min(per_tok, 4096 / T));
  const dim3 grid(T, gy);
  if (f32)
    hipLaunchKernelGGL((qkv_rope_cache_kernel<float>), grid, dim3(NT), 0, stream, (const float*)qkv, stride, bias,
                       positions, cos_sin, Hq, Hkv, dim, vdim, rot_dims, interleaved, unit, eps, v_first, v_mode, lam,
                       slots, (float*)cache, bs, (float*)q_out, qk_w, norm_first, v_from_k);
  else if (dim % 8 == 0 && dim <= 512 && ((dim >> 3) & ((dim >> 3) - 1)) == 0 && stride % 8 == 0 &&
           rot_dims % (interleaved ? 8 : 16) == 0 &&
           (((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)cache | (uintptr_t)bias | (uintptr_t)cos_sin) & 15) == 0) {
    // a pass covers 256 / (dim / 8) heads: fewer workgroups per token than the element-wise form
    const int hpp = NT / (dim >> 3);
    const int per_tok_v = (Hq + Hkv + hpp - 1) / hpp;
    const dim3 vgrid(T, std::max(1, std::min(per_tok_v, 4096 / T)));
    hipLaunchKernelGGL(qkv_rope_cache_vec_kernel, vgrid, dim3(NT), 0, stream, (const bf16_t*)qkv, stride, bias, positions,
                       cos_sin, Hq, Hkv, dim, vdim, rot_dims, interleaved, unit, eps, v_first, v_mode, lam, slots,
                       (bf16_t*)cache, bs, (bf16_t*)q_out, qk_w, norm_first, v_from_k);
  } else
    hipLaunchKernelGGL((qkv_rope_cache_kernel<bf16_t>), grid, dim3(NT), 0, stream, (const bf16_t*)qkv, stride, bias,
                       positions, cos_sin, Hq, Hkv, dim, vdim, rot_dims, interleaved, unit, eps, v_first, v_mode, lam,
                       slots, (bf16_t*)cache, bs, (bf16_t*)q_out, qk_w, norm_first, v_from_k);
}

// Returns 0, or 1 when the sizes do not fit the kernel (vdim > 1024 or rows too wide for LDS).
int sm_grouped_attention(const void* q, const void* cache, const int* tables, int W, int bs, const int* row_seq,
                         const int* row_len, float scale, int Hq, int Hkv, int dim, int vdim, int T, int QT,
                         const void* gate, int64_t gate_stride, void* out, int f32, const float* slopes, int chunk,
                         const float* sinks, int window, int keep, hipStream_t stream) {
  if (T == 0) return 0;
  const int vc = (vdim + 63) / 64;
#define SM_GO(TYPE, VC)                                                                                          \
  return launch_attn<TYPE, VC>(q, cache, tables, W, bs, row_seq, row_len, scale, Hq, Hkv, dim, vdim, T, QT, gate, \
                               gate_stride, out, slopes, chunk, sinks, window, keep, stream)
  if (f32) {
    if (vc <= 1) SM_GO(float, 1);
    if (vc <= 2) SM_GO(float, 2);
    if (vc <= 4) SM_GO(float, 4);
    if (vc <= 8) SM_GO(float, 8);
    if (vc <= 16) SM_GO(float, 16);
  } else {
    if (vc <= 1) SM_GO(bf16_t, 1);
    if (vc <= 2) SM_GO(bf16_t, 2);
    if (vc <= 4) SM_GO(bf16_t, 4);
    if (vc <= 8) SM_GO(bf16_t, 8);
    if (vc <= 16) SM_GO(bf16_t, 16);
  }
#undef SM_GO
  return 1;
}

// bf16, matrix cores. ``rb`` (1 or 2): blocks of 16 rows per wave - items hold up to 64 rb rows;
// key ranges (nsplit > 1) need rb = 1. Returns 0, or 1 when the sizes are outside the compiled forms
// (dim > 256, vdim > 256, group size > 64).
int sm_grouped_attention_mfma(const void* q, const void* cache, const int* tables, int W, int bs, const int* items,
                              int n_items, const int* row_len, float scale, int Hq, int Hkv, int dim, int vdim,
                              const void* gate, int64_t gate_stride, void* out, int nsplit, int split_keys,
                              float* part_o, float* part_ml, int rb, const float* slopes, int chunk,
                              const float* sinks, int window, int keep, hipStream_t stream) {
  if (n_items == 0) return 0;
  const int nks = (dim + 31) / 32, ncb = (vdim + 15) / 16;
  if (Hq / Hkv > 64 || nks > 8 || ncb > 16 || (rb != 1 && rb != 2) || (nsplit > 1 && rb != 1) || bs % 8) return 1;
  if (n_items > 65535) return 1;
  const dim3 grid(Hkv, n_items, nsplit);
#define SM_GO(NKS, NCB, RB)                                                                                       \
  hipLaunchKernelGGL((grouped_attention_mfma_kernel<NKS, NCB, RB>), grid, dim3(NT), 0, stream, (const bf16_t*)q,   \
                     (const bf16_t*)cache, tables, W, bs, items, row_len, scale, Hq, Hkv, dim, vdim,               \
                     (const bf16_t*)gate, gate_stride, (bf16_t*)out, split_keys, part_o, part_ml, slopes, chunk, \
                     sinks, window, keep)
#define SM_GO2(NKS, NCB) \
  if (rb == 2) SM_GO(NKS, NCB, 2); \
  else SM_GO(NKS, NCB, 1)
  if (nks <= 2 && ncb <= 4) { SM_GO2(2, 4); }
  else if (nks <= 4 && ncb <= 8) { SM_GO2(4, 8); }
  else { SM_GO2(8, 16); }
#undef SM_GO2
#undef SM_GO
  if (nsplit > 1)
    hipLaunchKernelGGL(grouped_attention_merge_kernel, dim3(n_items, Hkv, 64), dim3(NT), 0, stream, items, nsplit,
                       part_o, part_ml, Hq, Hkv, vdim, (const bf16_t*)gate, gate_stride, (bf16_t*)out);
  return 0;
}

}  // extern "C"
