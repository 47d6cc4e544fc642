// Gated delta rule over a step's per-sequence token runs (seq_start [n+1]), each continuing the
// state in its slot (seq_slot) or starting from zero (seq_init == 0). The state S [dk, dv] per head
// is fp32.
//
//   q, k <- unit vectors (x / sqrt(sum x^2 + 1e-6)), q times dk^-1/2
//   g = exp(-A_h softplus(a + dt_bias))   one per head, or one per head and key channel (row of S)
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//   out = o / rms(o) * norm_w * gate,  gate = silu or sigmoid of its input
//
// One workgroup per (value head, sequence): CT column threads (a multiple of 64 >= dv) x NW key
// groups. Thread (g, j) keeps the KR = KD / NW key rows [g KR, (g + 1) KR) of column j of S in
// registers (KD >= dk, padded rows stay zero). Per token the first dk threads compute the key-side
// vectors (unit key, unit query, decay) in fp32 and broadcast them through LDS; every group forms its
// part of S^T k and, after the update, of S^T q, and the parts meet in LDS. The inputs of a block of
// TB tokens are fetched while the previous block runs.
#include "seqmix_common.h"

using namespace sm;

namespace {

// Two sums over a workgroup of BT threads in one pass; every thread gets both.
template <int BT>
__device__ __forceinline__ void block_sum2(float& a, float& b, float* red) {
  a = wave_sum(a);
  b = wave_sum(b);
  if ((threadIdx.x & 63) == 0) {
    red[(threadIdx.x >> 6) * 2] = a;
    red[(threadIdx.x >> 6) * 2 + 1] = b;
  }
  __syncthreads();
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int i = 0; i < BT / 64; ++i) {
    sa += red[2 * i];
    sb += red[2 * i + 1];
  }
  __syncthreads();
  a = sa;
  b = sb;
}

template <typename T, int KD, int CT, int NW>
__global__ __launch_bounds__(CT * NW) void gated_delta_scan_kernel(
    const T* __restrict__ xc, int64_t x_stride, int G, int dk, int H, int dv, const T* __restrict__ beta_raw,
    int64_t beta_stride, const T* __restrict__ decay_raw, int64_t decay_stride, int per_channel,
    const float* __restrict__ A, const float* __restrict__ dt_bias, const T* __restrict__ gate_raw,
    int64_t gate_stride, int gate_sigmoid, const T* __restrict__ norm_w, float eps, float* __restrict__ state,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot, const int* __restrict__ seq_init,
    T* __restrict__ out) {
  constexpr int BT = CT * NW, KR = KD / NW;
  __shared__ __attribute__((aligned(16))) float sk[KD], sq[KD], sg[KD];
  __shared__ float part[NW][CT];
  __shared__ float red[2 * (BT / 64)];
  const int h = blockIdx.x, s = blockIdx.y;
  const int tid = threadIdx.x;
  const int j = tid % CT, g = tid / CT;
  const bool col = j < dv;
  const bool keyl = tid < dk;                 // this thread owns key channel tid of the token
  const bool lead = g == 0 && col;            // this thread writes column j of the output
  const int qh = h / (H / G);                 // the query / key head of this value head
  const int lo = seq_start[s], hi = seq_start[s + 1];
  float* sp = state + ((int64_t)seq_slot[s] * H + h) * dk * dv;
  const int i0 = g * KR;
  float S[KR];
  const bool init = seq_init[s] != 0;
#pragma unroll
  for (int i = 0; i < KR; ++i) S[i] = (col && i0 + i < dk && init) ? sp[(int64_t)(i0 + i) * dv + j] : 0.f;
  for (int i = dk + tid; i < KD; i += BT) {
    sk[i] = sq[i] = 0.f;
    sg[i] = 1.f;
  }
  const float Ah = A[h];
  const int dch = per_channel ? h * dk + (keyl ? tid : 0) : h;  // this thread's decay column
  const float dtb = dt_bias[dch];
  const float nwj = col ? ld(norm_w + j) : 0.f;
  const float qscale = 1.f / sqrtf((float)dk);
  const int nqk = G * dk;
  constexpr int TB = 4;
  float nq[TB], nk[TB], na[TB], nv[TB], nb[TB], ng[TB];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      nq[b] = nk[b] = na[b] = nv[b] = ng[b] = 0.f;
      const int t = min(t0 + b, hi - 1);  // past the end: a valid row, never used
      const T* xr = xc + (int64_t)t * x_stride;
      nb[b] = ld(beta_raw + (int64_t)t * beta_stride + h);
      if (keyl) {
        nq[b] = ld(xr + qh * dk + tid);
        nk[b] = ld(xr + nqk + qh * dk + tid);
        na[b] = ld(decay_raw + (int64_t)t * decay_stride + dch);
      }
      if (col) nv[b] = ld(xr + 2 * nqk + h * dv + j);
      if (lead) ng[b] = ld(gate_raw + (int64_t)t * gate_stride + h * dv + j);
    }
  };
  if (lo < hi) fetch(lo);
  for (int t0 = lo; t0 < hi; t0 += TB) {
    float cq[TB], ck[TB], ca[TB], cv[TB], cb[TB], cg[TB];
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      cq[b] = nq[b];
      ck[b] = nk[b];
      ca[b] = na[b];
      cv[b] = nv[b];
      cb[b] = nb[b];
      cg[b] = ng[b];
    }
    if (t0 + TB < hi) fetch(t0 + TB);
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      const int t = t0 + b;
      if (t >= hi) break;
      float ssq = keyl ? cq[b] * cq[b] : 0.f, ssk = keyl ? ck[b] * ck[b] : 0.f;
      block_sum2<BT>(ssq, ssk, red);  // also fences the previous token's LDS reads
      if (keyl) {
        sq[tid] = cq[b] * Fn<T>::rsqrt(ssq + 1e-6f) * qscale;
        sk[tid] = ck[b] * Fn<T>::rsqrt(ssk + 1e-6f);
        sg[tid] = Fn<T>::exp(-Ah * Fn<T>::softplus(ca[b] + dtb));
      }
      __syncthreads();
      // the key-side vectors come as 16-byte LDS broadcasts; entries beyond dk are 0 (decay 1)
      float pred = 0.f;
#pragma unroll
      for (int i = 0; i < KR; i += 4) {
        const float4 g4 = *reinterpret_cast<const float4*>(&sg[i0 + i]);
        const float4 k4 = *reinterpret_cast<const float4*>(&sk[i0 + i]);
        S[i] *= g4.x;
        S[i + 1] *= g4.y;
        S[i + 2] *= g4.z;
        S[i + 3] *= g4.w;
        pred += k4.x * S[i] + k4.y * S[i + 1] + k4.z * S[i + 2] + k4.w * S[i + 3];
      }
      if (NW > 1) {
        part[g][j] = pred;
        __syncthreads();
        pred = 0.f;
#pragma unroll
        for (int q = 0; q < NW; ++q) pred += part[q][j];
        __syncthreads();
      }
      const float u = Fn<T>::sigmoid(cb[b]) * (cv[b] - pred);
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < KR; i += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(&sk[i0 + i]);
        const float4 q4 = *reinterpret_cast<const float4*>(&sq[i0 + i]);
        S[i] += k4.x * u;
        S[i + 1] += k4.y * u;
        S[i + 2] += k4.z * u;
        S[i + 3] += k4.w * u;
        o += S[i] * q4.x + S[i + 1] * q4.y + S[i + 2] * q4.z + S[i + 3] * q4.w;
      }
      if (NW > 1) {
        part[g][j] = o;
        __syncthreads();
        o = 0.f;
#pragma unroll
        for (int q = 0; q < NW; ++q) o += part[q][j];
      }
      const float ss = block_sum<BT>(lead ? o * o : 0.f, red);
      if (lead) {
        const float gt = gate_sigmoid ? Fn<T>::sigmoid(cg[b]) : Fn<T>::silu(cg[b]);
        st(out + (int64_t)t * H * dv + h * dv + j, o * Fn<T>::rsqrt(ss / (float)dv + eps) * nwj * gt);
      }
    }
  }
  if (col && hi > lo) {
#pragma unroll
    for (int i = 0; i < KR; ++i)
      if (i0 + i < dk) sp[(int64_t)(i0 + i) * dv + j] = S[i];
  }
}

}  // namespace

extern "C" {

// Returns 0, or 1 when a head size does not fit (dk > 256 or dv > 256).
int sm_gated_delta_scan(const void* xc, int64_t x_stride, int G, int dk, int H, int dv, const void* beta_raw,
                        int64_t beta_stride, const void* decay_raw, int64_t decay_stride, int per_channel,
                        const float* A, const float* dt_bias, const void* gate_raw, int64_t gate_stride,
                        int gate_sigmoid, const void* norm_w, float eps, float* state, const int* seq_start,
                        const int* seq_slot, const int* seq_init, void* out, int nseq, int f32, hipStream_t stream) {
  if (nseq == 0) return 0;
  if (dk > 256 || dv > 256) return 1;
  const dim3 grid(H, nseq);
#define SM_GO(TYPE, KD, CT, NW)                                                                                     \
  hipLaunchKernelGGL((gated_delta_scan_kernel<TYPE, KD, CT, NW>), grid, dim3(CT * NW), 0, stream, (const TYPE*)xc,   \
                     x_stride, G, dk, H, dv, (const TYPE*)beta_raw, beta_stride, (const TYPE*)decay_raw,             \
                     decay_stride, per_channel, A, dt_bias, (const TYPE*)gate_raw, gate_stride, gate_sigmoid,        \
                     (const TYPE*)norm_w, eps, state, seq_start, seq_slot, seq_init, (TYPE*)out)
#define SM_KD(TYPE, CT, NW)                    \
  if (dk <= 32) SM_GO(TYPE, 32, CT, NW);       \
  else if (dk <= 64) SM_GO(TYPE, 64, CT, NW);  \
  else if (dk <= 128) SM_GO(TYPE, 128, CT, NW); \
  else SM_GO(TYPE, 256, CT, NW)
#define SM_CT(TYPE)                       \
  if (dv <= 64) { SM_KD(TYPE, 64, 4); }   \
  else if (dv <= 128) { SM_KD(TYPE, 128, 2); } \
  else { SM_KD(TYPE, 256, 2); }
  if (f32) { SM_CT(float) }
  else { SM_CT(bf16_t) }
#undef SM_CT
#undef SM_KD
#undef SM_GO
  return 0;
}

}  // extern "C"
