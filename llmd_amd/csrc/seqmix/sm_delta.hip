// Gated delta rule over a step's per-sequence token runs (seq_start [n+1]), each continuing the
// state in its slot (seq_slot) or starting from zero (seq_init == 0). The state S [dk, dv] per head
// is fp32.
//
//   q, k <- unit vectors (x / sqrt(sum x^2 + 1e-6)), q times dk^-1/2
//   g = exp(-A_h softplus(a + dt_bias))   one per head, or one per head and key channel (row of S)
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//   out = o / rms(o) * norm_w * gate,  gate = silu or sigmoid of its input
//
// Only the recurrence is sequential, so it is all the scan kernel does. A first kernel, parallel
// over the tokens, makes the unit queries and keys, the decays and beta (fp32, rows padded to
// KD = 32 .. 256 with q = k = 0 and g = 1); a last one, parallel again, norms the read-outs and applies
// the gate. The columns of S never meet in the recurrence, so the scan has no barrier: a workgroup
// is ONE wave that owns 16 (or 8) value columns of one head and sequence, lane = (column c, row group
// r of 4 (or 8)), and keeps rows [r KR, (r + 1) KR) of its column in registers. The two sums over the
// key rows (S^T k and S^T q) end with DPP exchanges between the lanes of a column. The key-side
// vectors reach the wave in blocks of tokens through LDS, fetched a block ahead. Steps with few
// (head, sequence) pairs - a prompt - take the 8 x 8 form: twice the waves, half the work of each.
#include "seqmix_common.h"
#include <algorithm>

using namespace sm;

namespace {

constexpr int NT = 256;

// Unit queries and keys, decays and beta of every token (fp32). qn, kn [T, G, KD]; dec [T, H, KD]
// (one decay per key channel) or [T, H]; beta [T, H]. Rows beyond dk: q = k = 0, g = 1.
template <typename T>
__global__ __launch_bounds__(NT) void delta_prep_kernel(const T* __restrict__ xc, int64_t x_stride, int G, int dk,
                                                       int KD, int H, const T* __restrict__ beta_raw,
                                                       int64_t beta_stride, const T* __restrict__ decay_raw,
                                                       int64_t decay_stride, int per_channel,
                                                       const float* __restrict__ A, const float* __restrict__ dt_bias,
                                                       float* __restrict__ qn, float* __restrict__ kn,
                                                       float* __restrict__ dec, float* __restrict__ beta) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* xr = xc + t * x_stride;
  const float qscale = 1.f / sqrtf((float)dk);
  for (int hd = wave; hd < 2 * G; hd += NT / 64) {  // q heads, then k heads: back to back in the row
    float r[4], ss = 0.f;                           // KD <= 256
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = lane + 64 * i;
      r[i] = e < dk ? ld(xr + hd * dk + e) : 0.f;
      ss += r[i] * r[i];
    }
    const float inv = Fn<T>::rsqrt(wave_sum(ss) + 1e-6f) * (hd < G ? qscale : 1.f);
    float* dst = (hd < G ? qn + (t * G + hd) * KD : kn + (t * G + hd - G) * KD);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = lane + 64 * i;
      if (e < KD) dst[e] = r[i] * inv;
    }
  }
  if (per_channel) {
    for (int idx = threadIdx.x; idx < H * KD; idx += NT) {
      const int h = idx / KD, i = idx - h * KD;
      float g = 1.f;
      if (i < dk) g = Fn<T>::exp(-A[h] * Fn<T>::softplus(ld(decay_raw + t * decay_stride + h * dk + i) + dt_bias[h * dk + i]));
      dec[t * H * KD + idx] = g;
    }
  }
  for (int h = threadIdx.x; h < H; h += NT) {
    if (!per_channel) dec[t * H + h] = Fn<T>::exp(-A[h] * Fn<T>::softplus(ld(decay_raw + t * decay_stride + h) + dt_bias[h]));
    beta[t * H + h] = Fn<T>::sigmoid(ld(beta_raw + t * beta_stride + h));
  }
}

// HGRN2: queries, gates and write strengths of every token (fp32), from the projection [q | f | ...].
// qn = silu(q), dec = f = lower + (1 - lower) sigmoid(f_raw + bias), kn = 1 - f; all [T, H, KD].
// Rows beyond dk: q = k = 0, f = 1.
template <typename T>
__global__ __launch_bounds__(NT) void hgrn2_prep_kernel(const T* __restrict__ p, int64_t p_stride, int H, int dk,
                                                       int KD, const float* __restrict__ f_bias,
                                                       const float* __restrict__ lower, float* __restrict__ qn,
                                                       float* __restrict__ kn, float* __restrict__ dec) {
  const int64_t t = blockIdx.x;
  const T* pr = p + t * p_stride;
  for (int idx = blockIdx.y * NT + threadIdx.x; idx < H * KD; idx += gridDim.y * NT) {
    const int h = idx / KD, i = idx - h * KD;
    float q = 0.f, k = 0.f, f = 1.f;
    if (i < dk) {
      const int c = h * dk + i;
      q = Fn<T>::silu(ld(pr + c));
      const float lo = lower[c];
      const float sg = Fn<T>::sigmoid(ld(pr + H * dk + c) + f_bias[c]);
      f = lo + (1.f - lo) * sg;
      k = (1.f - lo) * (1.f - sg);  // 1 - f without the cancellation near f = 1
    }
    qn[t * H * KD + idx] = q;
    kn[t * H * KD + idx] = k;
    dec[t * H * KD + idx] = f;
  }
}

// Sum over the RG (4 or 8) neighbouring lanes of a column (lanes RG c .. RG c + RG - 1): DPP
// exchanges, no LDS. After the two quad exchanges all four lanes of a quad hold the quad's sum; the
// mirror inside a half row (lane i <-> 7 - i) then brings the other quad's.
template <int RG>
__device__ __forceinline__ float group_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));  // 1 0 3 2
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));  // 2 3 0 1
  if (RG == 8)
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // half mirror
  return v;
}

// The recurrence. One wave per (head, block of 64 / RG value columns, sequence); RG = 4 or 8 row groups
// (lanes) per column, KR rows per lane. CH: a decay per key row.
// The key-side vectors of TB tokens at a time go through LDS: while the wave computes one block of
// tokens from one buffer, the next block's loads are in flight into registers, and are written to the
// other buffer afterwards - the recurrence never waits for global memory. Per token a lane reads its
// KR rows of k, q (and g) as 16-byte LDS broadcasts.
// OUT = false: the state alone is advanced (no read-out) - the first pass of the chunked form below.
template <typename T, int KR, int RG, bool CH, int TB, bool DELTA = true, bool OUT = true>
__global__ __launch_bounds__(64) void gated_delta_scan_kernel(
    const float* __restrict__ qn, const float* __restrict__ kn, const float* __restrict__ dec,
    const float* __restrict__ beta, const T* __restrict__ xc, int64_t x_stride, int voff, int G, int dk, int H, int dv,
    float* __restrict__ state, const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_init, float* __restrict__ o_raw, float* __restrict__ run_decay = nullptr) {
  constexpr int KD = RG * KR, CPW = 64 / RG, NV = CH ? 3 : 2;       // vectors per token: k, q (, g)
  constexpr int C4 = KD / 4;                         // 16-byte chunks per vector
  constexpr int NL = TB * NV * C4 / 64;              // chunks per lane and block (KD >= 32: a whole number)
  __shared__ __attribute__((aligned(16))) float buf[2][TB * NV * KD];
  const int ncb = (dv + CPW - 1) / CPW;
  const int h = blockIdx.x / ncb, cb = blockIdx.x - h * ncb, s = blockIdx.y;
  const int lane = threadIdx.x, r = lane % RG, c = lane / RG;
  const int col = cb * CPW + c;
  const bool colok = col < dv;
  const int qh = h / (H / G);
  const int row0 = r * KR;
  const int lo = seq_start[s], hi = seq_start[s + 1];
  if (lo >= hi) return;
  float* sp = state + ((int64_t)seq_slot[s] * H + h) * dk * dv;
  const bool init = seq_init[s] != 0;
  float S[KR];
#pragma unroll
  for (int i = 0; i < KR; ++i) S[i] = (init && colok && row0 + i < dk) ? sp[(int64_t)(row0 + i) * dv + col] : 0.f;
  // pass 1 of the chunked form: the waves of a head's first column block also multiply the run's decays
  const bool want_decay = !OUT && CH && run_decay != nullptr && cb == 0;
  float D[(!OUT && CH) ? KR : 1];
#pragma unroll
  for (int i = 0; i < ((!OUT && CH) ? KR : 1); ++i) D[i] = 1.f;
  // one token: kp, qp, gp point at this lane's KR rows of k, q and (CH) g; returns the read-out
  auto token = [&](const float4* kp, const float4* qp, const float4* gp, float gj, float bj, float vj) {
    float k[KR];
    float p[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < KR; i += 4) {
      const float4 k4 = kp[i >> 2];
      k[i] = k4.x; k[i + 1] = k4.y; k[i + 2] = k4.z; k[i + 3] = k4.w;
      if (CH) {
        const float4 g4 = gp[i >> 2];
        S[i] *= g4.x; S[i + 1] *= g4.y; S[i + 2] *= g4.z; S[i + 3] *= g4.w;
        if (!OUT && want_decay) {
          D[i] *= g4.x; D[i + 1] *= g4.y; D[i + 2] *= g4.z; D[i + 3] *= g4.w;
        }
      } else {
        S[i] *= gj; S[i + 1] *= gj; S[i + 2] *= gj; S[i + 3] *= gj;
      }
      if (DELTA) {
        p[0] += k[i] * S[i];
        p[1] += k[i + 1] * S[i + 1];
        p[2] += k[i + 2] * S[i + 2];
        p[3] += k[i + 3] * S[i + 3];
      }
    }
    const float pred = DELTA ? group_sum<RG>((p[0] + p[1]) + (p[2] + p[3])) : 0.f;
    const float u = DELTA ? bj * (vj - pred) : vj;
    float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < KR; i += 4) {
      const float4 q4 = qp[i >> 2];
      S[i] += k[i] * u; S[i + 1] += k[i + 1] * u; S[i + 2] += k[i + 2] * u; S[i + 3] += k[i + 3] * u;
      if (OUT) {
        o[0] += S[i] * q4.x;
        o[1] += S[i + 1] * q4.y;
        o[2] += S[i + 2] * q4.z;
        o[3] += S[i + 3] * q4.w;
      }
    }
    return OUT ? group_sum<RG>((o[0] + o[1]) + (o[2] + o[3])) : 0.f;
  };
  if (hi - lo <= 2) {
    // a decoded token (or two): the lane's rows straight from global memory, no staging
    for (int64_t t = lo; t < hi; ++t) {
      const float4* kp = reinterpret_cast<const float4*>(kn + (t * G + qh) * KD + row0);
      const float4* qp = reinterpret_cast<const float4*>(qn + (t * G + qh) * KD + row0);
      const float4* gp = reinterpret_cast<const float4*>(CH ? dec + (t * H + h) * KD + row0 : kn);
      const float vj = colok ? ld(xc + t * x_stride + voff + h * dv + col) : 0.f;
      const float ov = token(kp, qp, gp, CH ? 1.f : dec[t * H + h], DELTA ? beta[t * H + h] : 1.f, vj);
      if (OUT && r == 0 && colok) o_raw[t * H * dv + h * dv + col] = ov;
    }
  } else {
    float4 stage[NL];
    float vb[TB], bb[TB], gb[CH ? 1 : TB];            // the block's values, betas and per-head decays
    auto fetch = [&](int t0) {                          // block t0 .. t0 + TB - 1 -> registers
#pragma unroll
      for (int n = 0; n < NL; ++n) {
        const int e = lane + 64 * n;
        const int j = e / (NV * C4), rem = e - j * (NV * C4);
        const int var = rem / C4, i4 = rem - var * C4;
        const int64_t t = t0 + j;
        float4 v4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (t < hi) {
          const float* src =
              var == 0 ? kn + (t * G + qh) * KD : var == 1 ? qn + (t * G + qh) * KD : dec + (t * H + h) * KD;
          v4 = reinterpret_cast<const float4*>(src)[i4];
        }
        stage[n] = v4;
      }
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        const int64_t t = t0 + j;
        vb[j] = bb[j] = 0.f;
        if (!CH) gb[j] = 1.f;
        if (t >= hi) continue;
        vb[j] = colok ? ld(xc + t * x_stride + voff + h * dv + col) : 0.f;
        bb[j] = DELTA ? beta[t * H + h] : 1.f;
        if (!CH) gb[j] = dec[t * H + h];
      }
    };
    auto spill = [&](int which) {                       // registers -> LDS buffer
#pragma unroll
      for (int n = 0; n < NL; ++n) reinterpret_cast<float4*>(buf[which])[lane + 64 * n] = stage[n];
    };
    fetch(lo);
    spill(0);
    __syncthreads();
    int which = 0;
    for (int t0 = lo; t0 < hi; t0 += TB, which ^= 1) {
      float cv[TB], cbeta[TB], cg[CH ? 1 : TB];
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        cv[j] = vb[j];
        cbeta[j] = bb[j];
        if (!CH) cg[j] = gb[j];
      }
      const bool more = t0 + TB < hi;
      if (more) fetch(t0 + TB);
      const float* bk = buf[which];
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        if (t0 + j >= hi) break;
        const float ov = token(reinterpret_cast<const float4*>(bk + (j * NV + 0) * KD + row0),
                               reinterpret_cast<const float4*>(bk + (j * NV + 1) * KD + row0),
                               reinterpret_cast<const float4*>(bk + (j * NV + (CH ? 2 : 0)) * KD + row0),
                               CH ? 1.f : cg[j], cbeta[j], cv[j]);
        if (OUT && r == 0 && colok) o_raw[(int64_t)(t0 + j) * H * dv + h * dv + col] = ov;
      }
      if (more) spill(which ^ 1);
      __syncthreads();  // one wave: orders the buffer's writes before the next block's reads
    }
  }
  if (colok) {
#pragma unroll
    for (int i = 0; i < KR; ++i)
      if (row0 + i < dk) sp[(int64_t)(row0 + i) * dv + col] = S[i];
  }
  if (!OUT && CH && want_decay && c == 0) {
#pragma unroll
    for (int i = 0; i < KR; ++i) run_decay[((int64_t)s * H + h) * KD + row0 + i] = D[i];
  }
}

// Chunked form of the recurrence without the delta term, for prompts: S <- diag(g) S + k v^T is linear in
// S, so a run cut into chunks can be scanned in all chunks at once. Pass 1 scans every chunk from zero
// (its own contribution L_c, no read-out) and multiplies the chunk's decays (D_c, one per key row); the
// small kernel below walks a sequence's chunks in order, S_(c+1) = D_c S_c + L_c, leaving every
// chunk's true start state where its L_c was and the run's final state in the sequence's slot; pass 2
// scans every chunk again from its start state and reads out. All fp32; against the token-by-token scan
// only the order of the additions that form a chunk's start state differs.
// c_state [chunks, H, dk, dv]: in L_c, out the start state of chunk c. s_chunk0 [nseq + 1] bounds each
// sequence's chunks.
__global__ __launch_bounds__(NT) void chunk_link_kernel(float* __restrict__ c_state, const float* __restrict__ c_decay,
                                                       const int* __restrict__ s_chunk0, int H, int dk, int dv, int KD,
                                                       float* __restrict__ state, const int* __restrict__ seq_slot,
                                                       const int* __restrict__ seq_init) {
  const int s = blockIdx.y;
  const int64_t n = (int64_t)H * dk * dv;
  const int c0 = s_chunk0[s], c1 = s_chunk0[s + 1];
  if (c0 >= c1) return;
  float* sp = state + (int64_t)seq_slot[s] * n;
  const bool init = seq_init[s] != 0;
  for (int64_t e = (int64_t)blockIdx.x * NT + threadIdx.x; e < n; e += (int64_t)gridDim.x * NT) {
    const int h = (int)(e / ((int64_t)dk * dv)), i = (int)((e / dv) % dk);
    float S = init ? sp[e] : 0.f;
    for (int c = c0; c < c1; ++c) {
      const float own = c_state[(int64_t)c * n + e];
      c_state[(int64_t)c * n + e] = S;
      S = c_decay[((int64_t)c * H + h) * KD + i] * S + own;
    }
    sp[e] = S;
  }
}

// out = o / rms(o) * norm_w * gate per head; a wave per (token, head), any dv.
template <typename T>
__global__ __launch_bounds__(NT) void delta_out_kernel(const float* __restrict__ o_raw, const T* __restrict__ gate_raw,
                                                      int64_t gate_stride, int gate_sigmoid,
                                                      const T* __restrict__ norm_w, float eps, int H, int dv,
                                                      T* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int h = blockIdx.y * (NT / 64) + wave; h < H; h += gridDim.y * (NT / 64)) {
    const float* orow = o_raw + (t * H + h) * dv;
    float ss = 0.f;
    for (int e = lane; e < dv; e += 64) ss += orow[e] * orow[e];
    const float inv = Fn<T>::rsqrt(wave_sum(ss) / (float)dv + eps);
    for (int e = lane; e < dv; e += 64) {
      float gt = 1.f;  // no gate: the norm alone
      if (gate_raw != nullptr) {
        const float gr = ld(gate_raw + t * gate_stride + h * dv + e);
        gt = gate_sigmoid ? Fn<T>::sigmoid(gr) : Fn<T>::silu(gr);
      }
      st(out + (t * H + h) * dv + e, orow[e] * inv * ld(norm_w + e) * gt);
    }
  }
}

}  // namespace

extern "C" {

// Padded key rows per head (4 KR) for a key size, or 0 when it does not fit (dk > 256).
int sm_gated_delta_rows(int dk) { return dk <= 32 ? 32 : dk <= 64 ? 64 : dk <= 128 ? 128 : dk <= 256 ? 256 : 0; }

// Workspaces (fp32): qn, kn [T, G, KD]; dec [T, H, KD] or [T, H]; beta [T, H]; o_raw [T, H, dv].
// Returns 0, or 1 when the key size does not fit (dk > 256).
int sm_gated_delta_scan(const void* xc, int64_t x_stride, int G, int dk, int H, int dv, const void* beta_raw,
                        int64_t beta_stride, const void* decay_raw, int64_t decay_stride, int per_channel,
                        const float* A, const float* dt_bias, const void* gate_raw, int64_t gate_stride,
                        int gate_sigmoid, const void* norm_w, float eps, float* state, const int* seq_start,
                        const int* seq_slot, const int* seq_init, void* out, float* qn, float* kn, float* dec,
                        float* beta, float* o_raw, int T, int nseq, int f32, hipStream_t stream) {
  if (nseq == 0 || T == 0) return 0;
  const int KD = sm_gated_delta_rows(dk);
  if (KD == 0) return 1;
  const int voff = 2 * G * dk;
  // 16 columns x 4 row groups per wave when the step brings many waves anyway (decode: 64-byte pieces of
  // the state's rows); 8 x 8 when it brings few (a prompt): twice the waves, half the work of each
  const bool wide = (int64_t)nseq * H * ((dv + 15) / 16) >= 1024;
  const int cpw = wide ? 16 : 8;
  const dim3 grid(H * ((dv + cpw - 1) / cpw), nseq);
  const dim3 ogrid(T, std::max(1, std::min((H + 3) / 4, 4096 / T)));
#define SM_GO(TYPE, KR, RG, CH)                                                                                     \
  hipLaunchKernelGGL((gated_delta_scan_kernel<TYPE, KR, RG, CH, (KR * RG <= 128 ? 16 : 8)>), grid, dim3(64), 0, stream, \
                     qn, kn, dec, beta, (const TYPE*)xc, x_stride, voff, G, dk, H, dv, state, seq_start, seq_slot,  \
                     seq_init, o_raw)
#define SM_RG(TYPE, KD_, CH)              \
  if (wide) SM_GO(TYPE, KD_ / 4, 4, CH);  \
  else SM_GO(TYPE, KD_ / 8, 8, CH)
#define SM_KR(TYPE, CH)                           \
  if (KD == 32) { SM_RG(TYPE, 32, CH); }          \
  else if (KD == 64) { SM_RG(TYPE, 64, CH); }     \
  else if (KD == 128) { SM_RG(TYPE, 128, CH); }   \
  else { SM_RG(TYPE, 256, CH); }
#define SM_ALL(TYPE)                                                                                                \
  hipLaunchKernelGGL((delta_prep_kernel<TYPE>), dim3(T), dim3(NT), 0, stream, (const TYPE*)xc, x_stride, G, dk, KD, \
                     H, (const TYPE*)beta_raw, beta_stride, (const TYPE*)decay_raw, decay_stride, per_channel, A,   \
                     dt_bias, qn, kn, dec, beta);                                                                   \
  if (per_channel) { SM_KR(TYPE, true) }                                                                           \
  else { SM_KR(TYPE, false) }                                                                                      \
  hipLaunchKernelGGL((delta_out_kernel<TYPE>), ogrid, dim3(NT), 0, stream, o_raw, (const TYPE*)gate_raw,            \
                     gate_stride, gate_sigmoid, (const TYPE*)norm_w, eps, H, dv, (TYPE*)out)
  if (f32) { SM_ALL(float); }
  else { SM_ALL(bf16_t); }
#undef SM_ALL
#undef SM_KR
#undef SM_RG
#undef SM_GO
  return 0;
}

// HGRN2 over the projection p = [q | f | v] (H dk, H dk, H dv columns). Workspaces (fp32): qn, kn, dec
// [T, H, KD]; o_raw [T, H, dv]. Returns 0, or 1 when the key size does not fit (dk > 256).
// nc > 0: the chunked form. c_start [nc + 1] bounds the chunks (every run cut into pieces), c_slot = 0 .. nc - 1,
// c_zero / c_one [nc] are all 0 / all 1, s_chunk0 [nseq + 1] bounds each sequence's chunks; c_state
// [nc, H, dk, dv] and c_decay [nc, H, KD] are fp32 scratch.
int sm_hgrn2_scan(const void* p, int64_t p_stride, int H, int dk, int dv, const float* f_bias, const float* lower,
                  const void* norm_w, float eps, float* state, const int* seq_start, const int* seq_slot,
                  const int* seq_init, void* out, float* qn, float* kn, float* dec, float* o_raw, int T, int nseq,
                  int f32, int nc, const int* c_start, const int* c_slot, const int* c_zero, const int* c_one,
                  const int* s_chunk0, float* c_state, float* c_decay, hipStream_t stream) {
  if (nseq == 0 || T == 0) return 0;
  const int KD = sm_gated_delta_rows(dk);
  if (KD == 0) return 1;
  const int voff = 2 * H * dk;
  const int nrun = nc > 0 ? nc : nseq;  // runs the scan kernel sees
  const bool wide = (int64_t)nrun * H * ((dv + 15) / 16) >= 1024;
  const int cpw = wide ? 16 : 8;
  const dim3 grid(H * ((dv + cpw - 1) / cpw), nrun);
  const dim3 pgrid(T, std::max(1, std::min((H * KD + NT - 1) / NT, 4096 / T)));
  const dim3 ogrid(T, std::max(1, std::min((H + 3) / 4, 4096 / T)));
#define SM_GO(TYPE, KR, RG, OUT_, ST, START, SLOT, INIT)                                                              \
  hipLaunchKernelGGL((gated_delta_scan_kernel<TYPE, KR, RG, true, (KR * RG <= 128 ? 16 : 8), false, OUT_>), grid,      \
                     dim3(64), 0, stream, qn, kn, dec, nullptr, (const TYPE*)p, p_stride, voff, H, dk, H, dv, ST,      \
                     START, SLOT, INIT, o_raw, c_decay)
#define SM_RG(TYPE, KD_, ...)                      \
  if (wide) SM_GO(TYPE, KD_ / 4, 4, __VA_ARGS__);  \
  else SM_GO(TYPE, KD_ / 8, 8, __VA_ARGS__)
#define SM_KD(TYPE, ...)                                     \
  if (KD == 32) { SM_RG(TYPE, 32, __VA_ARGS__); }            \
  else if (KD == 64) { SM_RG(TYPE, 64, __VA_ARGS__); }       \
  else if (KD == 128) { SM_RG(TYPE, 128, __VA_ARGS__); }     \
  else { SM_RG(TYPE, 256, __VA_ARGS__); }
#define SM_ALL(TYPE)                                                                                                 \
  hipLaunchKernelGGL((hgrn2_prep_kernel<TYPE>), pgrid, dim3(NT), 0, stream, (const TYPE*)p, p_stride, H, dk, KD,      \
                     f_bias, lower, qn, kn, dec);                                                                    \
  if (nc > 0) {                                                                                                      \
    SM_KD(TYPE, false, c_state, c_start, c_slot, c_zero)                                                             \
    hipLaunchKernelGGL(chunk_link_kernel, dim3((unsigned)std::min<int64_t>(((int64_t)H * dk * dv + NT - 1) / NT, 2048), \
                                               nseq), dim3(NT), 0, stream, c_state, c_decay, s_chunk0, H, dk, dv, KD, \
                       state, seq_slot, seq_init);                                                                   \
    SM_KD(TYPE, true, c_state, c_start, c_slot, c_one)                                                               \
  } else {                                                                                                           \
    SM_KD(TYPE, true, state, seq_start, seq_slot, seq_init)                                                          \
  }                                                                                                                  \
  hipLaunchKernelGGL((delta_out_kernel<TYPE>), ogrid, dim3(NT), 0, stream, o_raw, (const TYPE*)nullptr, (int64_t)0, 0, \
                     (const TYPE*)norm_w, eps, H, dv, (TYPE*)out)
  if (f32) { SM_ALL(float); }
  else { SM_ALL(bf16_t); }
#undef SM_ALL
#undef SM_KD
#undef SM_RG
#undef SM_GO
  return 0;
}

}  // extern "C"
