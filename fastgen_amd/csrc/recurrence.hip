// A linear recurrence with a decay per key channel (gated linear attention), token by token:
//
//   a_t = sigmoid(z_t + b)^(1/tau)                       (per head and key channel, fp32)
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T                  (per head, [d, e] fp32, kept per request)
//   o_t = S_t^T (q_t * q_scale)
//
// The state lives in fp32 in a slot per request and is carried from step to step; a step brings a
// run of tokens per sequence (one when decoding).  Every token's arithmetic is the same whatever the
// step holds besides it: the tokens of a sequence are taken in order, each output element is one
// fixed chain of additions, so a prompt cut into portions or batched with others gives the same bits.
//
// grid (B sequences, H heads, ceil(e / 16)); one wave.  Lane l owns value channel 16 z + (l & 15) and
// the key channels rg * rpl .. rg * rpl + rpl - 1 with rg = l >> 4, rpl = ceil(d / 4): a quarter of a
// column of S in registers.  q, k and the decays of a few tokens go through LDS.
#include "common.h"

#define RC_TOKENS 4  // tokens staged at a time

struct ScanArgs {
  const void* qkv; int row_stride, q_col, k_col, v_col;  // act dtype rows: q, k [H * d], v [H * e] at their columns
  const float* z; int z_stride;                          // fp32 [T, >= H * d]: the decay's logits before the bias
  const float* z_bias;                                   // fp32 [H * d] or null
  float inv_tau, q_scale;
  float* state;                                          // fp32 [n_slots, H, d, e]
  const int* slot_ids; const int* q_start;               // [B], [B + 1]
  float* out;                                            // fp32 [T, H * e]
  int H, d, e;
};

template <class TA, int RPL>
__global__ __launch_bounds__(FG_WAVE) void decay_scan_kernel(const ScanArgs a) {
  extern __shared__ float lds[];  // [RC_TOKENS][3][d]: decay, k, q
  const int lane = threadIdx.x;
  const int b = blockIdx.x, h = blockIdx.y;
  const int c = lane & 15, rg = lane >> 4;
  const int col = blockIdx.z * 16 + c;
  const bool col_ok = col < a.e;
  const int d = a.d, e = a.e;
  const int rpl = (d + 3) / 4;
  const int r0 = rg * rpl;
  const int t_begin = a.q_start[b], t_end = a.q_start[b + 1];
  float* S_mem = a.state + (((size_t)a.slot_ids[b] * a.H + h) * d) * e;
  float S[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int r = r0 + i;
    S[i] = (i < rpl && r < d && col_ok) ? S_mem[(size_t)r * e + col] : 0.f;
  }
  for (int t0 = t_begin; t0 < t_end; t0 += RC_TOKENS) {
    const int n = min(RC_TOKENS, t_end - t0);
    __syncthreads();
    for (int idx = lane; idx < n * d; idx += FG_WAVE) {
      const int tt = idx / d, r = idx % d;
      const size_t t = (size_t)(t0 + tt);
      float zv = a.z[t * a.z_stride + h * d + r];
      if (a.z_bias) zv += a.z_bias[h * d + r];
      // log sigmoid(z) = min(z, 0) - log1p(exp(-|z|)), then the power as a product in the exponent
      const float ls = fminf(zv, 0.f) - log1pf(expf(-fabsf(zv)));
      const TA* row = (const TA*)a.qkv + t * a.row_stride;
      float* dst = lds + (size_t)tt * 3 * d;
      dst[r] = expf(ls * a.inv_tau);
      dst[d + r] = to_f<TA>(row[a.k_col + h * d + r]);
      dst[2 * d + r] = to_f<TA>(row[a.q_col + h * d + r]) * a.q_scale;
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const size_t t = (size_t)(t0 + tt);
      const float* av = lds + (size_t)tt * 3 * d;
      const float* kv = av + d;
      const float* qv = kv + d;
      const float v = col_ok ? to_f<TA>(((const TA*)a.qkv)[t * a.row_stride + a.v_col + h * e + col]) : 0.f;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const int r = r0 + i;
        if (i < rpl && r < d) {
          S[i] = av[r] * S[i] + kv[r] * v;
          acc += S[i] * qv[r];
        }
      }
      // the four quarters of the column, in a fixed order
      const float a1 = __shfl(acc, c + 16, FG_WAVE), a2 = __shfl(acc, c + 32, FG_WAVE), a3 = __shfl(acc, c + 48, FG_WAVE);
      const float a0 = __shfl(acc, c, FG_WAVE);
      if (rg == 0 && col_ok) a.out[t * ((size_t)a.H * e) + h * e + col] = ((a0 + a1) + a2) + a3;
    }
  }
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int r = r0 + i;
    if (i < rpl && r < d && col_ok) S_mem[(size_t)r * e + col] = S[i];
  }
}

extern "C" int fg_decay_scan(const ScanArgs* args, int n_seqs, int act_dtype, hipStream_t stream) {
  if (n_seqs <= 0) return FG_OK;
  const ScanArgs& a = *args;
  if (a.H <= 0 || a.d <= 0 || a.d > 256 || a.e <= 0 || a.H > 65535 || (a.e + 15) / 16 > 65535 || !a.qkv || !a.z ||
      !a.state || !a.slot_ids || !a.q_start || !a.out || !(a.inv_tau > 0.f))
    return FG_ERR_ARG;
  dim3 grid(n_seqs, a.H, (a.e + 15) / 16);
  const size_t lds = (size_t)RC_TOKENS * 3 * a.d * sizeof(float);
  const int rpl = (a.d + 3) / 4;
#define GO(TA, RPL) decay_scan_kernel<TA, RPL><<<grid, FG_WAVE, lds, stream>>>(a)
#define LAUNCH(TA)               \
  do {                           \
    if (rpl <= 8) GO(TA, 8);     \
    else if (rpl <= 16) GO(TA, 16); \
    else if (rpl <= 32) GO(TA, 32); \
    else GO(TA, 64);             \
  } while (0)
  if (act_dtype == FG_F32) LAUNCH(float);
  else if (act_dtype == FG_BF16) LAUNCH(bf16_t);
  else return FG_ERR_ARG;
#undef LAUNCH
#undef GO
  return fg_launch_status();
}
