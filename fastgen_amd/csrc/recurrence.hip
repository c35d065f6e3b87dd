// A linear recurrence with a decay per key channel (gated linear attention), token by token:
//
//   a_t = sigmoid(z_t + b)^(1/tau)                       (per head and key channel, fp32; all tokens at once)
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T                  (per head, [d, e] fp32, kept per request)
//   o_t = S_t^T (q_t * q_scale)
//
// The state lives in fp32 in a slot per request and is carried from step to step; a step brings a
// run of tokens per sequence (one when decoding).  Every token's arithmetic is the same whatever the
// step holds besides it: the tokens of a sequence are taken in order, each output element is one
// fixed chain of additions, so a prompt cut into portions or batched with others gives the same bits
// (long runs of tokens may instead be scanned chunk by chunk, see below: the same within rounding).
//
// grid (B sequences, H heads, ceil(e / 8)); one wave.  Lane l owns value channel 8 z + (l & 7) and the
// key channels rg * rpl .. rg * rpl + rpl - 1 with rg = l >> 3, rpl = ceil(d / 8): an eighth of a column
// of S in registers.  q, k and the decays of a run of tokens go through LDS.
#include "common.h"

// tokens staged at a time: as many as leave the kernel's registers unspilled
#define RC_TOKENS_FOR(RPL) ((RPL) <= 8 ? 16 : (RPL) <= 32 ? 8 : 4)

struct ScanArgs {
  const void* qkv; int row_stride, q_col, k_col, v_col;  // act dtype rows: q, k [H * d], v [H * e] at their columns
  const float* decay; int decay_stride;                  // fp32 [T, >= H * d]: a_t (fg_decay_from_logits)
  float q_scale;
  float* state;                                          // fp32 [n_slots, H, d, e]
  const int* slot_ids; const int* q_start;               // [B], [B + 1]
  float* out;                                            // fp32 [T, H * e]
  int H, d, e;
  int write_out, write_state;                            // what a sequence leaves: its tokens' outputs, its last state
};

// The loop over a sequence's tokens is a chain: what it costs is how many instructions one link takes
// (a wave issues one every few clocks) and what it waits for.  So the loads of a run of RC_TOKENS tokens
// (4, 8 or 16; decays, k, q: d of each a token, spread over the lanes; and each lane's own value channel) are all
// issued into registers before the run before it is computed, and reach LDS (q scaled) when that is
// done: memory latency passes behind the arithmetic.  The decays come ready from a kernel of their own
// (exponentials and logarithms of every token at once, not in this chain).  RPL >= ceil(d / 8); NJ =
// ceil(d / 64) is the number of staged elements a lane holds of each of the three, per token.
template <class TA, int RPL>
__global__ __launch_bounds__(FG_WAVE) void decay_scan_kernel(const ScanArgs a) {
  constexpr int NJ = RPL >= 8 ? RPL / 8 : 1;
  constexpr int RC_TOKENS = RC_TOKENS_FOR(RPL);
  // [RC_TOKENS][3][d + 32]: decay, k, q; key channel r lies at r + 4 (r / rpl), so that the eight parts
  // that the lane groups read at once start in different banks and every part is 16-byte aligned
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int lane = threadIdx.x;
  const int b = blockIdx.x, h = blockIdx.y;
  const int c = lane & 7, rg = lane >> 3;
  const int col = blockIdx.z * 8 + c;
  const bool col_ok = col < a.e;
  const int d = a.d, e = a.e;
  const int rpl = (d + 7) / 8;
  const int r0 = rg * rpl;
  const int ds = d + 32;              // a staged vector's stride
  const bool vec = rpl % 4 == 0 && d == 8 * rpl;  // uniform: the parts are read as float4
  const int t_begin = a.q_start[b], t_end = a.q_start[b + 1];
  float* S_mem = a.state + (((size_t)a.slot_ids[b] * a.H + h) * d) * e;
  float S[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int r = r0 + i;
    S[i] = (i < rpl && r < d && col_ok) ? S_mem[(size_t)r * e + col] : 0.f;
  }
  const TA* qkv = (const TA*)a.qkv;
  // the key channels this lane stages (the same for every token): where they come from and where they go
  int src[NJ], dst[NJ];
  bool mine[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int r = lane + FG_WAVE * j;
    mine[j] = r < d;
    src[j] = h * d + min(r, d - 1);
    dst[j] = r + 4 * (r / rpl);
  }
  const int v_src = a.v_col + h * e + min(col, e - 1);
  float pa[RC_TOKENS][NJ], pk[RC_TOKENS][NJ], pq[RC_TOKENS][NJ], pv[RC_TOKENS];
  auto fetch = [&](int t0) {  // the run t0 .. t0 + n - 1 into registers: nothing waits here
    const int n = min(RC_TOKENS, t_end - t0);
#pragma unroll
    for (int tt = 0; tt < RC_TOKENS; ++tt) {
      const size_t t = (size_t)(t0 + min(tt, n - 1));  // (never conditional: beyond the run, its last token again)
      const TA* row = qkv + t * a.row_stride;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        pa[tt][j] = a.decay[t * a.decay_stride + src[j]];
        pk[tt][j] = to_f<TA>(row[a.k_col + src[j]]);
        pq[tt][j] = to_f<TA>(row[a.q_col + src[j]]);
      }
      pv[tt] = to_f<TA>(row[v_src]);
    }
  };
  if (t_begin < t_end) fetch(t_begin);
  for (int t0 = t_begin; t0 < t_end; t0 += RC_TOKENS) {
    const int n = min(RC_TOKENS, t_end - t0);
    __syncthreads();  // the run before has been read
    float v[RC_TOKENS];
#pragma unroll
    for (int tt = 0; tt < RC_TOKENS; ++tt) {
      v[tt] = pv[tt];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (mine[j]) {
          float* to = lds + (size_t)tt * 3 * ds + dst[j];
          to[0] = pa[tt][j];
          to[ds] = pk[tt][j];
          to[2 * ds] = pq[tt][j] * a.q_scale;
        }
      }
    }
    __syncthreads();
    if (t0 + RC_TOKENS < t_end) fetch(t0 + RC_TOKENS);  // in flight while this run is computed
    // One token after the other; the sums over the lane groups are taken for the whole run at once (the
    // lanes' exchange is the longest link of the chain: sixteen of them wait together).  Reading a token's
    // operands from LDS a token ahead into a second set of registers was measured slower (the registers spill).
    float acc[RC_TOKENS];
    const float* part0 = lds + r0 + 4 * rg;  // this lane group's part of a staged vector
    if (vec) {
#pragma unroll
      for (int tt = 0; tt < RC_TOKENS; ++tt) {
        const float* av = part0 + (size_t)tt * 3 * ds;
        // four sums side by side (channels u, u + 4, ..), added up at the end: no chain of dependent additions
        float part[4] = {0.f, 0.f, 0.f, 0.f};
        if (tt < n) {
#pragma unroll
          for (int i4 = 0; i4 < RPL / 4; ++i4) {
            if (4 * i4 < rpl) {
              const float4 a4 = ((const float4*)av)[i4], k4 = ((const float4*)(av + ds))[i4],
                           q4 = ((const float4*)(av + 2 * ds))[i4];
              const float aa[4] = {a4.x, a4.y, a4.z, a4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, qq[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
              for (int u = 0; u < 4; ++u) {
                S[4 * i4 + u] = aa[u] * S[4 * i4 + u] + kk[u] * v[tt];
                part[u] += S[4 * i4 + u] * qq[u];
              }
            }
          }
        }
        acc[tt] = (part[0] + part[1]) + (part[2] + part[3]);
      }
    } else {
#pragma unroll
      for (int tt = 0; tt < RC_TOKENS; ++tt) {
        const float* av = part0 + (size_t)tt * 3 * ds;
        float sum = 0.f;
        if (tt < n) {
#pragma unroll
          for (int i = 0; i < RPL; ++i) {
            if (i < rpl && r0 + i < d) {
              S[i] = av[i] * S[i] + av[ds + i] * v[tt];
              sum += S[i] * av[2 * ds + i];
            }
          }
        }
        acc[tt] = sum;
      }
    }
    // the eight parts of a column: a butterfly whose order of additions is the same in every lane
#pragma unroll
    for (int m = 8; m < FG_WAVE; m <<= 1) {
      float other[RC_TOKENS];
#pragma unroll
      for (int tt = 0; tt < RC_TOKENS; ++tt) other[tt] = __shfl_xor(acc[tt], m, FG_WAVE);
#pragma unroll
      for (int tt = 0; tt < RC_TOKENS; ++tt) acc[tt] += other[tt];
    }
    if (rg == 0 && col_ok && a.write_out) {
#pragma unroll
      for (int tt = 0; tt < RC_TOKENS; ++tt)
        if (tt < n) a.out[(size_t)(t0 + tt) * ((size_t)a.H * e) + h * e + col] = acc[tt];
    }
  }
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int r = r0 + i;
    if (i < rpl && r < d && col_ok && a.write_state) S_mem[(size_t)r * e + col] = S[i];
  }
}

// out[t, c] = sigmoid(z[t, c] + bias[c])^(1/tau) for c < width, as exp(log sigmoid(.) / tau) with
// log sigmoid(x) = min(x, 0) - log1p(exp(-|x|)); fp32.
__global__ __launch_bounds__(256) void decay_from_logits_kernel(const float* __restrict__ z, int z_stride,
                                                                const float* __restrict__ bias, float inv_tau,
                                                                float* __restrict__ out, int width) {
  const size_t t = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const float x = z[t * z_stride + c] + (bias ? bias[c] : 0.f);
  out[t * width + c] = expf((fminf(x, 0.f) - log1pf(expf(-fabsf(x)))) * inv_tau);
}

extern "C" int fg_decay_from_logits(const float* z, int z_stride, const float* bias, float inv_tau, float* out,
                                    int n_rows, int width, hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (width <= 0 || z_stride < width || !(inv_tau > 0.f) || !z || !out) return FG_ERR_ARG;
  for (int r0 = 0; r0 < n_rows; r0 += 65535) {
    const int nr = n_rows - r0 < 65535 ? n_rows - r0 : 65535;
    decay_from_logits_kernel<<<dim3((width + 255) / 256, nr), 256, 0, stream>>>(
        z + (size_t)r0 * z_stride, z_stride, bias, inv_tau, out + (size_t)r0 * width, width);
  }
  return fg_launch_status();
}

// ------------------------------------------------------------ long prompts, chunk by chunk
// A long run of tokens is cut into chunks that are scanned side by side: first every chunk from a zero
// state (fg_decay_scan on the chunks as if they were sequences, states only), then, chunk after chunk of a
// sequence, the state each chunk starts from (below), then every chunk again from its true start, for
// the outputs.  Twice the arithmetic, as many times the waves as a sequence has chunks.
//
// prod[c, j] = the product of decay[t, j] over chunk c's tokens (chunk_start[c] .. chunk_start[c + 1] - 1).
__global__ __launch_bounds__(256) void decay_chunk_product_kernel(const float* __restrict__ decay, int decay_stride,
                                                                  const int* __restrict__ chunk_start,
                                                                  float* __restrict__ prod, int width) {
  const int c = blockIdx.y, j = blockIdx.x * 256 + threadIdx.x;
  if (j >= width) return;
  float p = 1.f;
  for (int t = chunk_start[c]; t < chunk_start[c + 1]; ++t) p *= decay[(size_t)t * decay_stride + j];
  prod[(size_t)c * width + j] = p;
}

// chunks [H, d, e] per chunk holds what each chunk adds to a zero state; it leaves with the state each chunk
// starts from: for sequence b's chunks c = seq_chunk[b] .. seq_chunk[b + 1] - 1 in order,
// start(c) = S; S = prod[c] * S + chunks[c], from S = state[slot_ids[b]], which takes the last S.
__global__ __launch_bounds__(256) void decay_chunk_states_kernel(float* __restrict__ chunks, const float* __restrict__ prod,
                                                                 float* __restrict__ state, const int* __restrict__ slot_ids,
                                                                 const int* __restrict__ seq_chunk, int H, int d, int e) {
  const int b = blockIdx.y;
  const size_t per = (size_t)H * d * e;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;  // (head, key channel, value channel)
  if (i >= per) return;
  const size_t row = i / e;  // (head, key channel)
  float* S_mem = state + (size_t)slot_ids[b] * per + i;
  float S = *S_mem;
  for (int c = seq_chunk[b]; c < seq_chunk[b + 1]; ++c) {
    float* at = chunks + (size_t)c * per + i;
    const float add = *at;
    *at = S;
    S = prod[(size_t)c * H * d + row] * S + add;
  }
  *S_mem = S;
}

extern "C" int fg_decay_chunk_product(const float* decay, int decay_stride, const int* chunk_start, float* prod,
                                      int n_chunks, int width, hipStream_t stream) {
  if (n_chunks <= 0) return FG_OK;
  if (width <= 0 || decay_stride < width || n_chunks > 65535 || !decay || !chunk_start || !prod) return FG_ERR_ARG;
  decay_chunk_product_kernel<<<dim3((width + 255) / 256, n_chunks), 256, 0, stream>>>(decay, decay_stride, chunk_start,
                                                                                      prod, width);
  return fg_launch_status();
}

extern "C" int fg_decay_chunk_states(float* chunks, const float* prod, float* state, const int* slot_ids,
                                     const int* seq_chunk, int n_seqs, int H, int d, int e, hipStream_t stream) {
  if (n_seqs <= 0) return FG_OK;
  const long long per = (long long)H * d * e;
  if (H <= 0 || d <= 0 || e <= 0 || n_seqs > 65535 || (per + 255) / 256 > 2147483647LL || !chunks || !prod || !state ||
      !slot_ids || !seq_chunk)
    return FG_ERR_ARG;
  decay_chunk_states_kernel<<<dim3((unsigned)((per + 255) / 256), n_seqs), 256, 0, stream>>>(chunks, prod, state, slot_ids,
                                                                                             seq_chunk, H, d, e);
  return fg_launch_status();
}

extern "C" int fg_decay_scan(const ScanArgs* args, int n_seqs, int act_dtype, hipStream_t stream) {
  if (n_seqs <= 0) return FG_OK;
  const ScanArgs& a = *args;
  if (a.H <= 0 || a.d <= 0 || a.d > 512 || a.e <= 0 || a.H > 65535 || (a.e + 7) / 8 > 65535 || !a.qkv || !a.decay ||
      !a.state || !a.slot_ids || !a.q_start || !a.out)
    return FG_ERR_ARG;
  dim3 grid(n_seqs, a.H, (a.e + 7) / 8);
  const int rpl = (a.d + 7) / 8;
#define GO(TA, RPL) \
  decay_scan_kernel<TA, RPL><<<grid, FG_WAVE, (size_t)RC_TOKENS_FOR(RPL) * 3 * (a.d + 32) * sizeof(float), stream>>>(a)
#define LAUNCH(TA)               \
  do {                           \
    if (rpl <= 4) GO(TA, 4);     \
    else if (rpl <= 8) GO(TA, 8);   \
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
