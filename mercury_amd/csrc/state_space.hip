// A state-space mixer (Mamba-2 make) in float32 arithmetic: the short causal convolution
// with its carried inputs, the recurrence over a step's tokens from the state earlier steps
// left, and the gated norm in groups behind it.
//
//   S_t = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T      (S is N x P per head)
//   y_t = S_t^T C_t + D_h x_t,   dt_t = softplus(raw_t + dt_bias_h)
//
// A step runs the tokens it brings, in order, sequence by sequence; nothing distinguishes a
// prompt portion from a decoded token, and the order of every sum depends on the sizes
// alone, so a position's result does not depend on how its sequence was cut.
//
// The recurrence: a workgroup of four wavefronts owns 32 columns p of one head of one
// sequence; a wavefront 8 columns x 8 slices of n, a lane a column and N/8 (padded to a
// multiple of 4) entries of n, so that the sum over n is in-lane but for three exchanges.
// B_t, C_t, x_t, dt_t and the decay of 16 tokens at a time are staged in LDS.  The state lies
// in memory as the lanes hold it ([head][block of 8 columns][entry][lane]), so reading and
// writing it is contiguous: a decoded token is one read and one write of the state.
#include <algorithm>

#include "common.h"
#include "mercury_kernels.h"

#define SS_TOKENS 16      // tokens staged at a time
#define SS_COLS 32        // columns of a workgroup
#define SS_MAX_NI 32      // entries of n a lane holds at most: N <= 256

namespace {

template <typename TW>
__device__ __forceinline__ float weight_at(const void* w, int i) {
  return Elem<TW>::load((const TW*)w + i);
}

__device__ __forceinline__ float silu_f(float v) { return v / (1.f + expf(-v)); }

// out[t, c] = silu(bias[c] + sum_j w[c, j] u(t - (taps-1) + j)[c]) over the sequence's own
// inputs u, those before this step's first token coming from `carried`
// [slot, taps - 1, channels] (oldest first; zeros in a fresh slot).
template <typename TW>
__global__ void causal_conv_kernel(const float* __restrict__ proj, int row_stride, int col0,
                                   int channels, int taps, const void* __restrict__ w,
                                   const void* __restrict__ bias,
                                   float* __restrict__ carried, size_t slot_stride,
                                   const int* __restrict__ slots,
                                   const int* __restrict__ token_seq,
                                   const int* __restrict__ cu_q, float* __restrict__ out) {
  const int t = blockIdx.x;
  const int seq = token_seq[t];
  const int local = t - cu_q[seq];
  // a sequence that brings one token (decoding) also moves its carried inputs on here: the
  // thread that read a channel's carried inputs is the only one that touches them
  const bool single = cu_q[seq + 1] - cu_q[seq] == 1;
  float* mine = carried + (size_t)slots[seq] * slot_stride;
  // a workgroup takes 256 channels of a token: few tokens still spread over the chip
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
    float acc = weight_at<TW>(bias, c);
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;            // how many tokens before t
      float u;
      if (back <= local) {
        u = proj[(size_t)(t - back) * row_stride + col0 + c];
      } else {
        // carried[k]: k = taps - 1 - (back - local)
        u = mine[(size_t)(taps - 1 - (back - local)) * channels + c];
      }
      acc = fmaf(weight_at<TW>(w, c * taps + j), u, acc);
    }
    out[(size_t)t * channels + c] = silu_f(acc);
    if (single && taps > 1) {
      for (int k = 0; k + 2 < taps; ++k) mine[(size_t)k * channels + c] = mine[(size_t)(k + 1) * channels + c];
      mine[(size_t)(taps - 2) * channels + c] = proj[(size_t)t * row_stride + col0 + c];
    }
  }
}

// After the convolution: the last taps - 1 inputs of every sequence of several tokens become
// its carried ones.
__global__ void conv_carry_kernel(const float* __restrict__ proj, int row_stride, int col0,
                                  int channels, int taps, float* __restrict__ carried,
                                  size_t slot_stride, const int* __restrict__ slots,
                                  const int* __restrict__ cu_q) {
  const int seq = blockIdx.x;
  const int first = cu_q[seq], count = cu_q[seq + 1] - first;
  if (count == 1) return;     // the convolution's own kernel moved this sequence's on
  float* mine = carried + (size_t)slots[seq] * slot_stride;
  const int keep = taps - 1;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
    // ascending k: entry k takes what entry k + count held, or this step's input
    for (int k = 0; k < keep; ++k) {
      const int at = count - keep + k;   // index among this step's tokens
      mine[(size_t)k * channels + c] =
          at >= 0 ? proj[(size_t)(first + at) * row_stride + col0 + c]
                  : mine[(size_t)(k + count) * channels + c];
    }
  }
}

// Long portions are cut into chunks of SS_CHUNK tokens that run side by side, in three passes:
// every chunk's recurrence from a zero state, which leaves the chunk's own contribution to
// the state at its end and the product of its decays (SS_LOCAL); one pass over the chunks of
// a sequence in order, S_in(k + 1) = decay(k) S_in(k) + local(k), from the state the slot
// holds, which leaves every chunk the state it starts from and the slot the last one
// (ssm_combine_kernel); and every chunk's recurrence again from that state, now with its
// outputs (SS_FROM).  Twice the arithmetic, for as many workgroups as there are chunks
// instead of one chain of dependent steps as long as the portion.  A step whose sequences all
// bring at most SS_CHUNK tokens (decoding) runs the recurrence once, slot to slot (SS_DIRECT).
enum { SS_DIRECT = 0, SS_LOCAL = 1, SS_FROM = 2 };
#define SS_CHUNK 128

__device__ __forceinline__ int chunks_of(int tokens) { return (tokens + SS_CHUNK - 1) / SS_CHUNK; }

// lane -> (column within the wavefront's 8, slice of n); entry i of a lane is
// n = (i / 4) * 32 + slice * 4 + i % 4, so that four entries are one 16-byte LDS read and the
// eight slices read 128 contiguous bytes.
// CPL: columns a lane holds (1 or 2).  With two, a wavefront owns 16 columns (two blocks of 8
// side by side in the state's layout) and reads B and C once for both: the LDS pipe, which the
// four SIMDs of a compute unit share, is what this loop waits for first.
template <int NI, typename TW, int MODE, int CPL>
__global__ __launch_bounds__(256) void ssm_scan_kernel(
    const float* __restrict__ xbc, int xbc_stride, const float* __restrict__ proj,
    int proj_stride, int z_col, int dt_col, const void* __restrict__ dt_bias,
    const void* __restrict__ a_log, const void* __restrict__ d_skip, float* __restrict__ state,
    size_t slot_stride, const int* __restrict__ slots, const int* __restrict__ cu_q, int heads,
    int P, int N, int groups, float* __restrict__ y_out, float* __restrict__ chunk_state,
    size_t chunk_stride, float* __restrict__ chunk_decay) {
  constexpr int NPAD = NI * 8;
  __shared__ __attribute__((aligned(16))) float sB[SS_TOKENS][NPAD];
  __shared__ __attribute__((aligned(16))) float sC[SS_TOKENS][NPAD];
  constexpr int COLS = SS_COLS * CPL;                   // columns of the workgroup
  __shared__ float sX[SS_TOKENS][COLS];
  __shared__ float sZ[SS_TOKENS][COLS];
  __shared__ float sDt[SS_TOKENS], sDecay[SS_TOKENS];

  const int head = blockIdx.y, pblock = blockIdx.x;
  int seq = blockIdx.z, first, count;
  if (MODE == SS_DIRECT) {
    first = cu_q[seq];
    count = cu_q[seq + 1] - first;
  } else {
    // chunk blockIdx.z of the step: the host launched as many as the sequences have together
    int chunk = blockIdx.z;
    seq = 0;
    for (int n = chunks_of(cu_q[1] - cu_q[0]); chunk >= n; n = chunks_of(cu_q[seq + 1] - cu_q[seq])) {
      chunk -= n;
      ++seq;
    }
    first = cu_q[seq] + chunk * SS_CHUNK;
    count = min(SS_CHUNK, cu_q[seq + 1] - first);
  }
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int slice = lane >> 3, col_in_wave = lane & 7;
  // column c of the lane is column (wave * CPL + c) * 8 + col_in_wave of the workgroup
  const int wave_col0 = pblock * COLS + wave * CPL * 8;
  const int group = head / (heads / groups);
  const int inner = heads * P;
  const int blocks8 = (P + SS_COLS - 1) / SS_COLS * (SS_COLS / 8);   // whole workgroups of 32

  const size_t within = ((size_t)head * blocks8 + (size_t)(pblock * 4 + wave) * CPL) * NI * 64;
  float* mine = MODE == SS_DIRECT ? state + (size_t)slots[seq] * slot_stride + within
                                  : chunk_state + (size_t)blockIdx.z * chunk_stride + within;
  bool live[CPL];                                       // the block of 8 has columns at all
  float S[CPL][NI];
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
    live[c] = wave_col0 + c * 8 < P;
#pragma unroll
    for (int i = 0; i < NI; ++i)
      S[c][i] = (MODE != SS_LOCAL && live[c]) ? mine[((size_t)c * NI + i) * 64 + lane] : 0.f;
  }

  const float rate = expf(weight_at<TW>(a_log, head));
  const float bias = weight_at<TW>(dt_bias, head);
  const float skip = weight_at<TW>(d_skip, head);
  float dt_sum = 0.f;

  for (int t0 = 0; t0 < count; t0 += SS_TOKENS) {
    const int n_tok = min(SS_TOKENS, count - t0);
    __syncthreads();
    for (int idx = tid; idx < n_tok * NPAD; idx += 256) {
      const int tt = idx / NPAD, n = idx - tt * NPAD;
      const float* row = xbc + (size_t)(first + t0 + tt) * xbc_stride + inner;
      sB[tt][n] = n < N ? row[group * N + n] : 0.f;
      if (MODE != SS_LOCAL) sC[tt][n] = n < N ? row[groups * N + group * N + n] : 0.f;
    }
    for (int idx = tid; idx < n_tok * COLS; idx += 256) {
      const int tt = idx / COLS, c = idx - tt * COLS;
      const int p = pblock * COLS + c;
      const size_t tok = first + t0 + tt;
      sX[tt][c] = p < P ? xbc[tok * xbc_stride + head * P + p] : 0.f;
      if (MODE != SS_LOCAL) sZ[tt][c] = p < P ? proj[tok * proj_stride + z_col + head * P + p] : 0.f;
    }
    if (tid < n_tok) {
      const float raw = proj[(size_t)(first + t0 + tid) * proj_stride + dt_col + head] + bias;
      // softplus without a clamp: log(1 + e^raw), written so that a large raw does not overflow
      const float dt = raw > 0.f ? raw + log1pf(expf(-raw)) : log1pf(expf(raw));
      sDt[tid] = dt;
      sDecay[tid] = expf(-rate * dt);
    }
    __syncthreads();
    for (int tt = 0; tt < n_tok; ++tt) {
      const float decay = sDecay[tt];
      float x[CPL], dtx[CPL];
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        x[c] = sX[tt][(wave * CPL + c) * 8 + col_in_wave];
        dtx[c] = sDt[tt] * x[c];
      }
      if (MODE == SS_LOCAL) {
        dt_sum += sDt[tt];
#pragma unroll
        for (int i4 = 0; i4 < NI / 4; ++i4) {
          const float4 b = *(const float4*)&sB[tt][i4 * 32 + slice * 4];
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
            float* s = &S[c][i4 * 4];
            s[0] = fmaf(decay, s[0], dtx[c] * b.x);
            s[1] = fmaf(decay, s[1], dtx[c] * b.y);
            s[2] = fmaf(decay, s[2], dtx[c] * b.z);
            s[3] = fmaf(decay, s[3], dtx[c] * b.w);
          }
        }
        continue;
      }
      // per column four sums side by side (entries i % 4), added up at the end:
      // ((y0 + y1) + (y2 + y3))
      float y0[CPL], y1[CPL], y2[CPL], y3[CPL];
#pragma unroll
      for (int c = 0; c < CPL; ++c) y0[c] = y1[c] = y2[c] = y3[c] = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < NI / 4; ++i4) {
        const float4 b = *(const float4*)&sB[tt][i4 * 32 + slice * 4];
        const float4 cc = *(const float4*)&sC[tt][i4 * 32 + slice * 4];
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
          float* s = &S[c][i4 * 4];
          s[0] = fmaf(decay, s[0], dtx[c] * b.x);
          s[1] = fmaf(decay, s[1], dtx[c] * b.y);
          s[2] = fmaf(decay, s[2], dtx[c] * b.z);
          s[3] = fmaf(decay, s[3], dtx[c] * b.w);
          y0[c] = fmaf(s[0], cc.x, y0[c]);
          y1[c] = fmaf(s[1], cc.y, y1[c]);
          y2[c] = fmaf(s[2], cc.z, y2[c]);
          y3[c] = fmaf(s[3], cc.w, y3[c]);
        }
      }
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        float y = (y0[c] + y1[c]) + (y2[c] + y3[c]);
        y += __shfl_xor(y, 8, MK_WAVE);
        y += __shfl_xor(y, 16, MK_WAVE);
        y += __shfl_xor(y, 32, MK_WAVE);
        const int col = wave_col0 + c * 8 + col_in_wave;   // column p of the head
        if (slice == 0 && col < P) {
          const float z = sZ[tt][(wave * CPL + c) * 8 + col_in_wave];
          y_out[(size_t)(first + t0 + tt) * inner + head * P + col] = (y + skip * x[c]) * silu_f(z);
        }
      }
    }
  }
  if (MODE != SS_FROM) {
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      if (!live[c]) continue;
#pragma unroll
      for (int i = 0; i < NI; ++i) mine[((size_t)c * NI + i) * 64 + lane] = S[c][i];
    }
  }
  if (MODE == SS_LOCAL && pblock == 0 && tid == 0) {
    chunk_decay[(size_t)blockIdx.z * heads + head] = expf(-rate * dt_sum);
  }
}

// The chunks of a sequence in order: chunk k's buffer holds what the chunk adds to the state
// and receives the state the chunk starts from; the slot receives the state after the last.
__global__ void ssm_combine_kernel(float* __restrict__ state, size_t slot_stride,
                                   const int* __restrict__ slots, const int* __restrict__ cu_q,
                                   float* __restrict__ chunk_state, size_t chunk_stride,
                                   const float* __restrict__ chunk_decay, int heads,
                                   size_t per_head) {
  const int seq = blockIdx.y;
  const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= per_head * heads) return;
  const int head = (int)(e / per_head);
  int chunk0 = 0;
  for (int s = 0; s < seq; ++s) chunk0 += chunks_of(cu_q[s + 1] - cu_q[s]);
  const int n = chunks_of(cu_q[seq + 1] - cu_q[seq]);
  float* slot = state + (size_t)slots[seq] * slot_stride;
  float run = slot[e];
  for (int k = 0; k < n; ++k) {
    float* at = chunk_state + (size_t)(chunk0 + k) * chunk_stride + e;
    const float local = *at;
    *at = run;
    run = fmaf(chunk_decay[(size_t)(chunk0 + k) * heads + head], run, local);
  }
  slot[e] = run;
}

// One workgroup per (token, part): out = y / rms(part of y) * weight.
template <typename T, typename TW>
__global__ void group_norm_kernel(const float* __restrict__ y, T* __restrict__ out,
                                  const void* __restrict__ weight, float eps, int width,
                                  int parts) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, part = blockIdx.y;
  const int size = width / parts;
  const float* src = y + (size_t)t * width + (size_t)part * size;
  float sq = 0.f;
  for (int i = threadIdx.x; i < size; i += blockDim.x) sq += src[i] * src[i];
  const float r = rsqrtf(block_sum(sq, scratch) / (float)size + eps);
  for (int i = threadIdx.x; i < size; i += blockDim.x) {
    Elem<T>::store(out + (size_t)t * width + (size_t)part * size + i,
                   src[i] * r * weight_at<TW>(weight, part * size + i));
  }
}

int entries_for(int N) {
  int ni = (N + 7) / 8;
  int padded = 4;
  while (padded < ni) padded *= 2;
  return padded;
}

}  // namespace

// Floats of recurrent state one head occupies, as the kernel lays it out.
extern "C" long long mk_ssm_state_floats(int heads, int P, int N) {
  if (heads <= 0 || P <= 0 || N <= 0 || N > SS_MAX_NI * 8) return -1;
  // whole workgroups of 32 columns, so that every wavefront's block exists
  const long long blocks8 = (long long)((P + SS_COLS - 1) / SS_COLS) * (SS_COLS / 8);
  return (long long)heads * blocks8 * entries_for(N) * 64;
}

extern "C" int mk_causal_conv_silu(const float* proj, int row_stride, int col0, int channels,
                                   int taps, const void* w, const void* bias, int weight_dtype,
                                   float* carried, long long slot_stride, const int* slots,
                                   const int* token_seq, const int* cu_q, float* out, int tokens,
                                   int num_seqs, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && num_seqs >= 0 && channels > 0 && taps >= 1, "causal_conv: bad sizes");
  MK_REQUIRE(col0 >= 0 && row_stride >= col0 + channels, "causal_conv: columns outside the row");
  MK_REQUIRE(slot_stride >= (long long)(taps - 1) * channels,
             "causal_conv: a slot of %lld floats does not hold %d x %d carried inputs",
             slot_stride, taps - 1, channels);
  MK_REQUIRE(weight_dtype == MK_F32 || weight_dtype == MK_BF16, "causal_conv: weight dtype %d",
             weight_dtype);
  if (tokens == 0) return 0;
  const int col_blocks = std::min(1024, (channels + 255) / 256);
  const dim3 grid(tokens, col_blocks);
  if (weight_dtype == MK_F32)
    causal_conv_kernel<float><<<grid, 256, 0, stream>>>(proj, row_stride, col0, channels, taps,
                                                           w, bias, carried, (size_t)slot_stride,
                                                           slots, token_seq, cu_q, out);
  else
    causal_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>(proj, row_stride, col0, channels, taps,
                                                            w, bias, carried, (size_t)slot_stride,
                                                            slots, token_seq, cu_q, out);
  MK_LAUNCH_CHECK("causal_conv");
  if (taps > 1 && tokens > num_seqs) {   // some sequence brings more than one token
    conv_carry_kernel<<<dim3(num_seqs, col_blocks), 256, 0, stream>>>(proj, row_stride, col0, channels, taps,
                                                    carried, (size_t)slot_stride, slots, cu_q);
    MK_LAUNCH_CHECK("conv_carry");
  }
  return 0;
}

// Tokens a chunk of the recurrence holds: a step with a longer sequence runs in chunks, and
// wants mk_ssm_scan_workspace floats of scratch memory for `total_chunks` of them.
extern "C" int mk_ssm_chunk_tokens() { return SS_CHUNK; }
extern "C" long long mk_ssm_scan_workspace(int total_chunks, int heads, int P, int N) {
  const long long per = mk_ssm_state_floats(heads, P, N);
  return per < 0 ? -1 : (long long)total_chunks * (per + heads);
}

extern "C" int mk_ssm_scan(const float* xbc, int xbc_stride, const float* proj, int proj_stride,
                           int z_col, int dt_col, const void* dt_bias, const void* a_log,
                           const void* d_skip, int weight_dtype, float* state,
                           long long slot_stride, const int* slots, const int* cu_q, int heads,
                           int P, int N, int groups, float* y_out, int tokens, int num_seqs,
                           int total_chunks, float* workspace, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && num_seqs >= 0 && heads > 0 && P > 0 && N > 0 && groups > 0,
             "ssm_scan: bad sizes");
  MK_REQUIRE(heads % groups == 0, "ssm_scan: %d heads are not a multiple of %d groups", heads, groups);
  MK_REQUIRE(N <= SS_MAX_NI * 8, "ssm_scan: state size %d exceeds %d", N, SS_MAX_NI * 8);
  const long long state_floats = mk_ssm_state_floats(heads, P, N);
  MK_REQUIRE(slot_stride >= state_floats,
             "ssm_scan: a slot of %lld floats does not hold the state", slot_stride);
  MK_REQUIRE(xbc_stride >= heads * P + 2 * groups * N, "ssm_scan: x, B, C outside the row");
  MK_REQUIRE(z_col >= 0 && dt_col >= 0 && proj_stride >= z_col + heads * P &&
                 proj_stride >= dt_col + heads, "ssm_scan: gate or step sizes outside the row");
  MK_REQUIRE(heads <= 65535 && num_seqs <= 65535, "ssm_scan: too many heads or sequences");
  MK_REQUIRE(weight_dtype == MK_F32 || weight_dtype == MK_BF16, "ssm_scan: weight dtype %d",
             weight_dtype);
  // total_chunks 0: every sequence brings at most a chunk's tokens, one pass slot to slot;
  // else the sum over the sequences of ceil(tokens / chunk), which the caller knows
  MK_REQUIRE(total_chunks == 0 || (total_chunks >= num_seqs && total_chunks <= 65535 && workspace &&
                                   (long long)total_chunks * SS_CHUNK >= tokens),
             "ssm_scan: %d chunks for %d tokens of %d sequences (or no workspace)", total_chunks,
             tokens, num_seqs);
  MK_REQUIRE(total_chunks != 0 || (long long)num_seqs * SS_CHUNK >= tokens,
             "ssm_scan: a sequence longer than a chunk runs in chunks");
  if (tokens == 0 || num_seqs == 0) return 0;
  // Two columns a lane where the head's workgroups of 32 columns come in pairs (the layout of
  // the state is the same either way) and a lane's registers hold twice the entries.
  const int blocks32 = (P + SS_COLS - 1) / SS_COLS;
  const int ni = entries_for(N);
  const int cpl = (blocks32 % 2 == 0 && ni <= 16) ? 2 : 1;
  const int pblocks = blocks32 / cpl;
  float* chunk_state = workspace;
  float* chunk_decay = workspace ? workspace + (size_t)total_chunks * state_floats : nullptr;
#define SS_RUN(NI, TW, MODE, grid)                                                              \
  if (cpl == 2)                                                                                 \
    ssm_scan_kernel<NI, TW, MODE, 2><<<grid, 256, 0, stream>>>(                                  \
        xbc, xbc_stride, proj, proj_stride, z_col, dt_col, dt_bias, a_log, d_skip, state,       \
        (size_t)slot_stride, slots, cu_q, heads, P, N, groups, y_out, chunk_state,              \
        (size_t)state_floats, chunk_decay);                                                     \
  else                                                                                          \
  ssm_scan_kernel<NI, TW, MODE, 1><<<grid, 256, 0, stream>>>(                                    \
      xbc, xbc_stride, proj, proj_stride, z_col, dt_col, dt_bias, a_log, d_skip, state,         \
      (size_t)slot_stride, slots, cu_q, heads, P, N, groups, y_out, chunk_state,                \
      (size_t)state_floats, chunk_decay)
#define SS_MODE(NI, MODE, grid)                                                                  \
  do {                                                                                          \
    if (weight_dtype == MK_F32) SS_RUN(NI, float, MODE, grid); else SS_RUN(NI, bf16_t, MODE, grid); \
  } while (0)
#define SS_LAUNCH(MODE, grid)                                                                    \
  do {                                                                                          \
    if (ni == 4) SS_MODE(4, MODE, grid);                                                         \
    else if (ni == 8) SS_MODE(8, MODE, grid);                                                    \
    else if (ni == 16) SS_MODE(16, MODE, grid);                                                  \
    else SS_MODE(32, MODE, grid);                                                                \
  } while (0)
  if (total_chunks == 0) {
    const dim3 grid(pblocks, heads, num_seqs);
    SS_LAUNCH(SS_DIRECT, grid);
    MK_LAUNCH_CHECK("ssm_scan");
    return 0;
  }
  const dim3 grid(pblocks, heads, total_chunks);
  SS_LAUNCH(SS_LOCAL, grid);
  MK_LAUNCH_CHECK("ssm_scan (chunks)");
  const size_t per_head = (size_t)(state_floats / heads);
  const dim3 cgrid((unsigned)((state_floats + 255) / 256), num_seqs);
  ssm_combine_kernel<<<cgrid, 256, 0, stream>>>(state, (size_t)slot_stride, slots, cu_q, chunk_state,
                                                (size_t)state_floats, chunk_decay, heads, per_head);
  MK_LAUNCH_CHECK("ssm_combine");
  SS_LAUNCH(SS_FROM, grid);
  MK_LAUNCH_CHECK("ssm_scan (outputs)");
#undef SS_LAUNCH
#undef SS_MODE
#undef SS_RUN
  return 0;
}

extern "C" int mk_group_rmsnorm(const float* y, void* out, int dtype, const void* weight,
                                int weight_dtype, float eps, int tokens, int width, int parts,
                                hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && width > 0 && parts > 0 && width % parts == 0,
             "group_rmsnorm: %d columns in %d parts", width, parts);
  MK_REQUIRE(parts <= 65535, "group_rmsnorm: too many parts");
  MK_REQUIRE(weight_dtype == MK_F32 || weight_dtype == MK_BF16, "group_rmsnorm: weight dtype %d",
             weight_dtype);
  if (tokens == 0) return 0;
  const dim3 grid(tokens, parts);
  const int size = width / parts;
  const int threads = size >= 1024 ? 256 : (size >= 256 ? 128 : 64);
#define GN_LAUNCH(T, TW)                                                            \
  group_norm_kernel<T, TW><<<grid, threads, 0, stream>>>(y, (T*)out, weight, eps, width, parts)
  if (dtype == MK_F32) {
    if (weight_dtype == MK_F32) GN_LAUNCH(float, float); else GN_LAUNCH(float, bf16_t);
  } else if (dtype == MK_BF16) {
    if (weight_dtype == MK_F32) GN_LAUNCH(bf16_t, float); else GN_LAUNCH(bf16_t, bf16_t);
  } else {
    MK_REQUIRE(false, "group_rmsnorm: unknown dtype %d", dtype);
  }
#undef GN_LAUNCH
  MK_LAUNCH_CHECK("group_rmsnorm");
  return 0;
}
