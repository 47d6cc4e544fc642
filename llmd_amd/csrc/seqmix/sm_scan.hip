// Recurrent mixers over a step's per-sequence token runs (seq_start [n+1]), each continuing the
// state in its slot (seq_slot) or starting from zero (seq_init == 0). States are fp32.
//
// causal_conv_silu : per-channel short convolution + SiLU; the last taps-1 inputs of a sequence
//                    are its convolution state (a second small kernel rolls it forward).
// input_conv       : h + conv(h), the same convolution without bias and activation, added to its input.
// selective_scan   : S[c,n] <- exp(dt_c A[c,n]) S[c,n] + dt_c x_c B_n; y_c = sum_n S[c,n] C_n + D_c x_c;
//                    y * silu(z). A channel's states sit in neighbouring lanes (groups of NL), the
//                    sum over n is a shuffle reduction; softplus, exp and the state are fp32.
// gdelta_scan      : S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r per head; one workgroup per
//                    (head, sequence), a thread owns one value column of S in registers, the token's
//                    key-side vectors are broadcast from LDS; then the head's RMS norm, weight and gate.
#include "seqmix_common.h"

using namespace sm;

namespace {

constexpr int NT = 256;

template <typename T>
__global__ __launch_bounds__(NT) void conv_silu_kernel(const T* __restrict__ xz, int64_t xz_stride, int C,
                                                      const T* __restrict__ w, const T* __restrict__ b, int taps,
                                                      const T* __restrict__ state, const int* __restrict__ seq_start,
                                                      const int* __restrict__ seq_slot,
                                                      const int* __restrict__ seq_init, T* __restrict__ out, int seg) {
  const int c = blockIdx.x * NT + threadIdx.x;
  const int s = blockIdx.y;
  const int lo = seq_start[s], hi = seq_start[s + 1];
  const int p0 = blockIdx.z * seg;
  if (c >= C || lo + p0 >= hi) return;
  const int p1 = min(hi - lo, p0 + seg);
  const bool init = seq_init[s] != 0;
  const T* st_ = state + (int64_t)seq_slot[s] * (taps - 1) * C;
  const float bias = ld(b + c);
  for (int p = p0; p < p1; ++p) {
    float a = bias;
    for (int j = 0; j < taps; ++j) {
      const int pp = p - (taps - 1 - j);  // the last tap is the current token's
      float v = 0.f;
      if (pp >= 0) v = ld(xz + (int64_t)(lo + pp) * xz_stride + c);
      else if (init) v = ld(st_ + (int64_t)(taps - 1 + pp) * C + c);
      a += ld(w + (int64_t)c * taps + j) * v;
    }
    st(out + (int64_t)(lo + p) * C + c, siluf_(a));
  }
}

// state[j] <- input at run position len - (taps-1) + j (from the run, or from the old state)
template <typename T>
__global__ __launch_bounds__(NT) void conv_state_kernel(const T* __restrict__ xz, int64_t xz_stride, int C, int taps,
                                                       T* __restrict__ state, const int* __restrict__ seq_start,
                                                       const int* __restrict__ seq_slot,
                                                       const int* __restrict__ seq_init, int skip_single = 0) {
  const int c = blockIdx.x * NT + threadIdx.x;
  const int s = blockIdx.y;
  if (c >= C) return;
  const int lo = seq_start[s], len = seq_start[s + 1] - lo;
  if (len <= 0 || (skip_single && len == 1)) return;  // a single token's roll was done where it was computed
  const bool init = seq_init[s] != 0;
  T* st_ = state + (int64_t)seq_slot[s] * (taps - 1) * C;
  for (int j = 0; j < taps - 1; ++j) {  // ascending j reads old entries j + len > j not yet rewritten
    const int pp = len - (taps - 1) + j;
    float v = 0.f;
    if (pp >= 0) v = ld(xz + (int64_t)(lo + pp) * xz_stride + c);
    else if (init) v = ld(st_ + (int64_t)(taps - 1 + pp) * C + c);
    st(st_ + (int64_t)j * C + c, v);
  }
}

// out = h + conv(h): one thread per (token, channel). The token's earlier inputs come from the run
// itself, from the sequence's state (its last taps - 1 inputs before this step) or are zero.
template <typename T>
__global__ __launch_bounds__(NT) void input_conv_kernel(const T* __restrict__ h, int C, const T* __restrict__ w,
                                                       int taps, T* state,
                                                       const int* __restrict__ row_seq,
                                                       const int* __restrict__ seq_start,
                                                       const int* __restrict__ seq_slot,
                                                       const int* __restrict__ seq_init, T* __restrict__ out) {
  const int c = blockIdx.y * NT + threadIdx.x;
  const int64_t t = blockIdx.x;
  if (c >= C) return;
  const int s = row_seq[t];
  const int p = (int)t - seq_start[s];  // place in the run
  const bool init = seq_init[s] != 0;
  T* st_ = state + (int64_t)seq_slot[s] * (taps - 1) * C;
  const float x = ld(h + t * C + c);
  float a = x + ld(w + (int64_t)c * taps + taps - 1) * x;
  for (int j = 0; j < taps - 1; ++j) {
    const int pp = p - (taps - 1 - j);
    float v = 0.f;
    if (pp >= 0) v = ld(h + (t - (taps - 1 - j)) * C + c);
    else if (init) v = ld(st_ + (int64_t)(taps - 1 + pp) * C + c);
    a += ld(w + (int64_t)c * taps + j) * v;
  }
  st(out + t * C + c, a);
  if (p == 0 && seq_start[s + 1] - seq_start[s] == 1) {
    // a run of one token (a decode step): nobody else reads or writes this sequence's state, so it is
    // rolled here; ascending j reads entry j + 1 before anything overwrites it
    for (int j = 0; j < taps - 2; ++j) st(st_ + (int64_t)j * C + c, init ? ld(st_ + (int64_t)(j + 1) * C + c) : 0.f);
    if (taps > 1) st(st_ + (int64_t)(taps - 2) * C + c, x);
  }
}

// bf16 form with 16-byte accesses: a thread owns eight neighbouring channels of one token and keeps their
// 8 x TAPS weights in registers (TAPS 16-byte loads: the weights of eight channels lie side by side).
// C a multiple of 8, TAPS <= 8.
constexpr int ICV_MAX_TAPS = 8;
template <int TAPS>
__global__ __launch_bounds__(NT) void input_conv_vec_kernel(const bf16_t* __restrict__ h, int C,
                                                           const bf16_t* __restrict__ w, bf16_t* state,
                                                           const int* __restrict__ row_seq,
                                                           const int* __restrict__ seq_start,
                                                           const int* __restrict__ seq_slot,
                                                           const int* __restrict__ seq_init,
                                                           bf16_t* __restrict__ out) {
  const int c = (blockIdx.y * NT + threadIdx.x) * 8;
  const int64_t t = blockIdx.x;
  if (c >= C) return;
  auto ld8 = [](const bf16_t* p, float* v) {
    const uint4 q = *reinterpret_cast<const uint4*>(p);
    v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xffff0000u);
    v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xffff0000u);
    v[4] = __uint_as_float(q.z << 16); v[5] = __uint_as_float(q.z & 0xffff0000u);
    v[6] = __uint_as_float(q.w << 16); v[7] = __uint_as_float(q.w & 0xffff0000u);
  };
  float wr[8 * TAPS];  // channel i, tap j at i * TAPS + j
#pragma unroll
  for (int i = 0; i < TAPS; ++i) ld8(w + (int64_t)c * TAPS + 8 * i, wr + 8 * i);
  const int s = row_seq[t];
  const int lo = seq_start[s];
  const int p = (int)t - lo;
  const bool init = seq_init[s] != 0;
  bf16_t* st_ = state + (int64_t)seq_slot[s] * (TAPS - 1) * C;
  float x[8], a[8];
  ld8(h + t * C + c, x);
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = x[i] + wr[i * TAPS + TAPS - 1] * x[i];
#pragma unroll
  for (int j = 0; j < TAPS - 1; ++j) {
    const int pp = p - (TAPS - 1 - j);
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (pp >= 0) ld8(h + (t - (TAPS - 1 - j)) * C + c, v);
    else if (init) ld8(st_ + (int64_t)(TAPS - 1 + pp) * C + c, v);
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] += wr[i * TAPS + j] * v[i];
  }
  uint4 o;
  auto pack = [](float lo_, float hi_) {
    const __bf16 l16 = (__bf16)lo_, h16 = (__bf16)hi_;
    return (uint32_t)__builtin_bit_cast(uint16_t, l16) | ((uint32_t)__builtin_bit_cast(uint16_t, h16) << 16);
  };
  o.x = pack(a[0], a[1]); o.y = pack(a[2], a[3]); o.z = pack(a[4], a[5]); o.w = pack(a[6], a[7]);
  *reinterpret_cast<uint4*>(out + t * C + c) = o;
  if (TAPS > 1 && p == 0 && seq_start[s + 1] - lo == 1) {  // a run of one token: its state is rolled here (see above)
    const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < TAPS - 2; ++j)
      *reinterpret_cast<uint4*>(st_ + (int64_t)j * C + c) =
          init ? *reinterpret_cast<const uint4*>(st_ + (int64_t)(j + 1) * C + c) : zero;
    *reinterpret_cast<uint4*>(st_ + (int64_t)(TAPS - 2) * C + c) = *reinterpret_cast<const uint4*>(h + t * C + c);
  }
}

// NL lanes per channel (power of two <= 64), SPL states per lane.
template <typename T, int SPL>
__global__ __launch_bounds__(NT) void selective_scan_kernel(
    const T* __restrict__ xc, const T* __restrict__ dt_raw, const T* __restrict__ dt_bias,
    const float* __restrict__ A, const T* __restrict__ bc, int64_t bc_stride, int R, int N, const T* __restrict__ D,
    const T* __restrict__ xz, int64_t xz_stride, int C, float* __restrict__ state, const int* __restrict__ seq_start,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_init, T* __restrict__ out, int NL) {
  const int cpb = NT / NL;
  const int c = blockIdx.x * cpb + threadIdx.x / NL;
  const int nl = threadIdx.x % NL;
  const int s = blockIdx.y;
  const int lo = seq_start[s], hi = seq_start[s + 1];
  const bool ok = c < C;
  const int cc = ok ? c : C - 1;  // idle lanes follow the last channel and store nothing
  float* sp = state + ((int64_t)seq_slot[s] * C + cc) * N;
  float S[SPL], Ac[SPL];
#pragma unroll
  for (int i = 0; i < SPL; ++i) {
    const int n = nl + i * NL;
    Ac[i] = n < N ? A[(int64_t)cc * N + n] : 0.f;
    S[i] = (n < N && seq_init[s]) ? sp[n] : 0.f;
  }
  const float bias = ld(dt_bias + cc), Dc = ld(D + cc);
  // inputs are fetched a block of TB tokens ahead of the recurrence: the loads of the next block
  // are in flight while this block's tokens run one after the other (memory latency is about one
  // token's worth of arithmetic, a single wave per SIMD cannot hide it otherwise)
  constexpr int TB = SPL <= 2 ? 8 : 4;
  float ndt[TB], nx[TB], nz[TB], nB[TB][SPL], nC[TB][SPL];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      const int t = min(t0 + b, hi - 1);  // past the end: a valid row, never used
      ndt[b] = ld(dt_raw + (int64_t)t * C + cc);
      nx[b] = ld(xc + (int64_t)t * C + cc);
      nz[b] = ld(xz + (int64_t)t * xz_stride + C + cc);
      const T* bt = bc + (int64_t)t * bc_stride + R;
#pragma unroll
      for (int i = 0; i < SPL; ++i) {
        const int n = nl + i * NL;
        nB[b][i] = n < N ? ld(bt + n) : 0.f;
        nC[b][i] = n < N ? ld(bt + N + n) : 0.f;
      }
    }
  };
  if (lo < hi) fetch(lo);
  for (int t0 = lo; t0 < hi; t0 += TB) {
    float cdt[TB], cx[TB], cz[TB], cB[TB][SPL], cC[TB][SPL];
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      cdt[b] = ndt[b];
      cx[b] = nx[b];
      cz[b] = nz[b];
#pragma unroll
      for (int i = 0; i < SPL; ++i) {
        cB[b][i] = nB[b][i];
        cC[b][i] = nC[b][i];
      }
    }
    if (t0 + TB < hi) fetch(t0 + TB);
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      const int t = t0 + b;
      if (t >= hi) break;
      const float dt = Fn<T>::softplus(cdt[b] + bias), x = cx[b];
      float part = 0.f;
#pragma unroll
      for (int i = 0; i < SPL; ++i) {
        const int n = nl + i * NL;
        if (n < N) {
          S[i] = Fn<T>::exp(dt * Ac[i]) * S[i] + dt * x * cB[b][i];
          part += S[i] * cC[b][i];
        }
      }
      for (int o = NL >> 1; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
      if (ok && nl == 0) st(out + (int64_t)t * C + c, (part + Dc * x) * Fn<T>::silu(cz[b]));
    }
  }
  if (ok) {
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      const int n = nl + i * NL;
      if (n < N) sp[n] = S[i];
    }
  }
}

constexpr float DECAY_K = 0.6065306597126334f;  // exp(-1/2)

// CT column threads (a multiple of 64 >= d) x NW key groups = 256 threads. Thread (g, j) keeps the
// KR = KD / NW key rows [g KR, (g + 1) KR) of column j of S in registers (KD >= d, padded rows stay
// zero). Per token: group 0 computes the key-side vectors (decay, removal rate x unit key, unit key,
// key, receptance) in fp32 and broadcasts them through LDS; every group forms its part of u^T S and,
// after the update, of S^T r, and the parts meet in LDS.
template <typename T, int KD, int CT, int NW>
__global__ __launch_bounds__(CT * NW) void gdelta_scan_kernel(
    const T* __restrict__ proj, int64_t p_stride, const T* __restrict__ wl, const T* __restrict__ w0,
    const T* __restrict__ a_b, const T* __restrict__ norm_w, float eps, int H, int d, float* __restrict__ state,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot, const int* __restrict__ seq_init,
    T* __restrict__ out) {
  constexpr int BT = CT * NW, KR = KD / NW;
  __shared__ __attribute__((aligned(16))) float sw[KD], sau[KD], su[KD], sk[KD], sr[KD];
  __shared__ float part[NW][CT];
  __shared__ float red[BT / 64];
  const int h = blockIdx.x, s = blockIdx.y;
  const int j = threadIdx.x % CT, g = threadIdx.x / CT;
  const bool col = j < d;
  const bool lead = g == 0 && col;
  const int HD = H * d;
  const int lo = seq_start[s], hi = seq_start[s + 1];
  float* sp = state + ((int64_t)seq_slot[s] * H + h) * d * d;
  const int i0 = g * KR;
  float S[KR];
  const bool init = seq_init[s] != 0;
#pragma unroll
  for (int i = 0; i < KR; ++i) S[i] = (col && i0 + i < d && init) ? sp[(int64_t)(i0 + i) * d + j] : 0.f;
  for (int i = d + threadIdx.x; i < KD; i += BT) sw[i] = sau[i] = su[i] = sk[i] = sr[i] = 0.f;
  const int e = h * d + (col ? j : 0);
  const float w0e = ld(w0 + e), abe = ld(a_b + e), nwe = ld(norm_w + e);
  // the inputs of this column are fetched a block of TB tokens ahead, so their latency overlaps the
  // previous block's arithmetic and barriers
  constexpr int TB = 4;
  float nk[TB], na[TB], nwl[TB], nr[TB], nv[TB], ng[TB];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      nk[b] = na[b] = nwl[b] = nr[b] = nv[b] = ng[b] = 0.f;
      const int t = min(t0 + b, hi - 1);  // past the end: a valid row, never used
      if (!col) continue;
      const T* pr = proj + (int64_t)t * p_stride;
      nv[b] = ld(pr + 2 * HD + e);
      if (g != 0) continue;
      nr[b] = ld(pr + e);
      nk[b] = ld(pr + HD + e);
      ng[b] = ld(pr + 3 * HD + e);
      na[b] = ld(pr + 4 * HD + e);
      nwl[b] = ld(wl + (int64_t)t * HD + e);
    }
  };
  if (lo < hi) fetch(lo);
  for (int t0 = lo; t0 < hi; t0 += TB) {
    float ck[TB], ca[TB], cwl[TB], cr_[TB], cv[TB], cg[TB];
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      ck[b] = nk[b];
      ca[b] = na[b];
      cwl[b] = nwl[b];
      cr_[b] = nr[b];
      cv[b] = nv[b];
      cg[b] = ng[b];
    }
    if (t0 + TB < hi) fetch(t0 + TB);
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      const int t = t0 + b;
      if (t >= hi) break;
      const float kj = ck[b], aj = ca[b], wlj = cwl[b], rj = cr_[b], v = cv[b], gj = cg[b];
      const float ksum = block_sum<BT>(lead ? kj * kj : 0.f, red);  // also fences the previous token's LDS reads
      if (lead) {
        const float u = kj * Fn<T>::rsqrt(ksum + 1e-6f);
        const float a = Fn<T>::sigmoid(aj + abe);
        sw[j] = Fn<T>::exp(-DECAY_K * Fn<T>::sigmoid(wlj + w0e));
        sau[j] = a * u;
        su[j] = u;
        sk[j] = kj;
        sr[j] = rj;
      }
      __syncthreads();
      // the key-side vectors come as 16-byte LDS broadcasts; entries beyond d are zero
      float sa = 0.f;
#pragma unroll
      for (int i = 0; i < KR; i += 4) {
        const float4 u4 = *reinterpret_cast<const float4*>(&su[i0 + i]);
        sa += u4.x * S[i] + u4.y * S[i + 1] + u4.z * S[i + 2] + u4.w * S[i + 3];
      }
      if (NW > 1) {
        part[g][j] = sa;
        __syncthreads();
        sa = 0.f;
#pragma unroll
        for (int q = 0; q < NW; ++q) sa += part[q][j];
        __syncthreads();
      }
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < KR; i += 4) {
        const float4 w4 = *reinterpret_cast<const float4*>(&sw[i0 + i]);
        const float4 a4 = *reinterpret_cast<const float4*>(&sau[i0 + i]);
        const float4 k4 = *reinterpret_cast<const float4*>(&sk[i0 + i]);
        const float4 r4 = *reinterpret_cast<const float4*>(&sr[i0 + i]);
        S[i] = w4.x * S[i] - a4.x * sa + k4.x * v;
        S[i + 1] = w4.y * S[i + 1] - a4.y * sa + k4.y * v;
        S[i + 2] = w4.z * S[i + 2] - a4.z * sa + k4.z * v;
        S[i + 3] = w4.w * S[i + 3] - a4.w * sa + k4.w * v;
        o += S[i] * r4.x + S[i + 1] * r4.y + S[i + 2] * r4.z + S[i + 3] * r4.w;
      }
      if (NW > 1) {
        part[g][j] = o;
        __syncthreads();
        o = 0.f;
#pragma unroll
        for (int q = 0; q < NW; ++q) o += part[q][j];
      }
      const float ss = block_sum<BT>(lead ? o * o : 0.f, red);
      if (lead) st(out + (int64_t)t * HD + e, o * Fn<T>::rsqrt(ss / (float)d + eps) * nwe * Fn<T>::sigmoid(gj));
    }
  }
  if (col) {
#pragma unroll
    for (int i = 0; i < KR; ++i)
      if (i0 + i < d) sp[(int64_t)(i0 + i) * d + j] = S[i];
  }
}

}  // namespace

extern "C" {

void sm_causal_conv_silu(const void* xz, int64_t xz_stride, int C, const void* w, const void* b, int taps, void* state,
                         const int* seq_start, const int* seq_slot, const int* seq_init, void* out, int nseq,
                         int max_q, int f32, hipStream_t stream) {
  if (nseq == 0 || max_q == 0) return;
  const int seg = 64;
  const dim3 g1((C + NT - 1) / NT, nseq, (max_q + seg - 1) / seg), g2((C + NT - 1) / NT, nseq);
  if (f32) {
    hipLaunchKernelGGL((conv_silu_kernel<float>), g1, dim3(NT), 0, stream, (const float*)xz, xz_stride, C,
                       (const float*)w, (const float*)b, taps, (const float*)state, seq_start, seq_slot, seq_init,
                       (float*)out, seg);
    if (taps > 1)
      hipLaunchKernelGGL((conv_state_kernel<float>), g2, dim3(NT), 0, stream, (const float*)xz, xz_stride, C, taps,
                         (float*)state, seq_start, seq_slot, seq_init);
  } else {
    hipLaunchKernelGGL((conv_silu_kernel<bf16_t>), g1, dim3(NT), 0, stream, (const bf16_t*)xz, xz_stride, C,
                       (const bf16_t*)w, (const bf16_t*)b, taps, (const bf16_t*)state, seq_start, seq_slot, seq_init,
                       (bf16_t*)out, seg);
    if (taps > 1)
      hipLaunchKernelGGL((conv_state_kernel<bf16_t>), g2, dim3(NT), 0, stream, (const bf16_t*)xz, xz_stride, C, taps,
                         (bf16_t*)state, seq_start, seq_slot, seq_init);
  }
}

// max_q: the longest run of the step; runs of one token roll their state in the first kernel, so a
// decode-only step needs no second launch.
void sm_input_conv(const void* h, int C, const void* w, int taps, void* state, const int* row_seq,
                   const int* seq_start, const int* seq_slot, const int* seq_init, void* out, int T, int nseq,
                   int max_q, int f32, hipStream_t stream) {
  if (nseq == 0 || T == 0) return;
  const dim3 g1(T, (C + NT - 1) / NT), g2((C + NT - 1) / NT, nseq);
  const bool roll = taps > 1 && max_q > 1;
  if (!f32 && C % 8 == 0 && taps <= ICV_MAX_TAPS &&
      (((uintptr_t)h | (uintptr_t)out | (uintptr_t)state | (uintptr_t)w) & 15) == 0) {
    const dim3 gv(T, (C / 8 + NT - 1) / NT);
#define SM_ICV(N)                                                                                                     \
  case N:                                                                                                             \
    hipLaunchKernelGGL(input_conv_vec_kernel<N>, gv, dim3(NT), 0, stream, (const bf16_t*)h, C, (const bf16_t*)w,      \
                       (bf16_t*)state, row_seq, seq_start, seq_slot, seq_init, (bf16_t*)out);                        \
    break
    switch (taps) {
      SM_ICV(1); SM_ICV(2); SM_ICV(3); SM_ICV(4); SM_ICV(5); SM_ICV(6); SM_ICV(7); SM_ICV(8);
    }
#undef SM_ICV
    if (roll)
      hipLaunchKernelGGL((conv_state_kernel<bf16_t>), g2, dim3(NT), 0, stream, (const bf16_t*)h, (int64_t)C, C, taps,
                         (bf16_t*)state, seq_start, seq_slot, seq_init, 1);
    return;
  }
  if (f32) {
    hipLaunchKernelGGL((input_conv_kernel<float>), g1, dim3(NT), 0, stream, (const float*)h, C, (const float*)w, taps,
                       (float*)state, row_seq, seq_start, seq_slot, seq_init, (float*)out);
    if (roll)
      hipLaunchKernelGGL((conv_state_kernel<float>), g2, dim3(NT), 0, stream, (const float*)h, (int64_t)C, C, taps,
                         (float*)state, seq_start, seq_slot, seq_init, 1);
  } else {
    hipLaunchKernelGGL((input_conv_kernel<bf16_t>), g1, dim3(NT), 0, stream, (const bf16_t*)h, C, (const bf16_t*)w,
                       taps, (bf16_t*)state, row_seq, seq_start, seq_slot, seq_init, (bf16_t*)out);
    if (roll)
      hipLaunchKernelGGL((conv_state_kernel<bf16_t>), g2, dim3(NT), 0, stream, (const bf16_t*)h, (int64_t)C, C, taps,
                         (bf16_t*)state, seq_start, seq_slot, seq_init, 1);
  }
}

// Returns 0, or 1 when the state size does not fit (N > 256).
int sm_selective_scan(const void* xc, const void* dt_raw, const void* dt_bias, const float* A, const void* bc,
                      int64_t bc_stride, int R, int N, const void* D, const void* xz, int64_t xz_stride, int C,
                      float* state, const int* seq_start, const int* seq_slot, const int* seq_init, void* out,
                      int nseq, int f32, hipStream_t stream) {
  if (nseq == 0) return 0;
  int NL = 1;
  while (NL < N && NL < 64) NL <<= 1;
  const int spl = (N + NL - 1) / NL;
  if (spl > 4) return 1;
  const dim3 grid((C + NT / NL - 1) / (NT / NL), nseq);
#define SM_GO(TYPE, SPL)                                                                                              \
  hipLaunchKernelGGL((selective_scan_kernel<TYPE, SPL>), grid, dim3(NT), 0, stream, (const TYPE*)xc,                  \
                     (const TYPE*)dt_raw, (const TYPE*)dt_bias, A, (const TYPE*)bc, bc_stride, R, N, (const TYPE*)D,  \
                     (const TYPE*)xz, xz_stride, C, state, seq_start, seq_slot, seq_init, (TYPE*)out, NL)
  if (f32) {
    if (spl == 1) SM_GO(float, 1);
    else if (spl == 2) SM_GO(float, 2);
    else SM_GO(float, 4);
  } else {
    if (spl == 1) SM_GO(bf16_t, 1);
    else if (spl == 2) SM_GO(bf16_t, 2);
    else SM_GO(bf16_t, 4);
  }
#undef SM_GO
  return 0;
}

// Returns 0, or 1 when the head size does not fit (d > 256).
int sm_gdelta_scan(const void* proj, int64_t p_stride, const void* wl, const void* w0, const void* a_b,
                   const void* norm_w, float eps, int H, int d, float* state, const int* seq_start,
                   const int* seq_slot, const int* seq_init, void* out, int nseq, int f32, hipStream_t stream) {
  if (nseq == 0) return 0;
  const dim3 grid(H, nseq);
#define SM_GO(TYPE, KD, CT, NW)                                                                                  \
  hipLaunchKernelGGL((gdelta_scan_kernel<TYPE, KD, CT, NW>), grid, dim3(CT * NW), 0, stream, (const TYPE*)proj,   \
                     p_stride, (const TYPE*)wl, (const TYPE*)w0, (const TYPE*)a_b, (const TYPE*)norm_w, eps, H, d, \
                     state, seq_start, seq_slot, seq_init, (TYPE*)out)
  if (f32) {
    if (d <= 32) SM_GO(float, 32, 64, 4);
    else if (d <= 64) SM_GO(float, 64, 64, 4);
    else if (d <= 128) SM_GO(float, 128, 128, 2);
    else if (d <= 256) SM_GO(float, 256, 256, 1);
    else return 1;
  } else {
    if (d <= 32) SM_GO(bf16_t, 32, 64, 4);
    else if (d <= 64) SM_GO(bf16_t, 64, 64, 4);
    else if (d <= 128) SM_GO(bf16_t, 128, 128, 2);
    else if (d <= 256) SM_GO(bf16_t, 256, 256, 1);
    else return 1;
  }
#undef SM_GO
  return 0;
}

}  // extern "C"
