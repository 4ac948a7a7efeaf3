// Attention through a low-rank latent: the per-token side of it, in float32 arithmetic.
//
// A token's keys and values of all heads are functions of one latent vector c (kv_rank wide)
// plus one rotated key part r (rot wide) shared by the heads, so c and r are all that is
// cached.  With W_uk[h] (dim x kv_rank) the matrix that would expand c into head h's
// unrotated key, the score of query head h against a cached token is
//     (W_uk[h]^T q_h) . c + q_rot_h . r
// and head h's value-weighted sum is W_uv[h] (sum_j p_j c_j).  So the attention itself is one
// shared key/value head of key width kv_rank + rot and value width kv_rank, which the paged
// attention kernels run; what is special lies around it and is here:
//
//   mk_latent_prepare     a token's down-projected row [q_rank | kv_rank | rot] (float32):
//                         RMS norm of the query latent (out, for the query up-projection), RMS
//                         norm of c, rotation of r, and the cache write: the key row [c | r]
//                         and, because the value-side product wants c with the keys as the fast
//                         index, c once more, transposed within the page.
//   mk_latent_query_tail  the rotated part of every query head, turned and placed behind the
//                         head's absorbed part (which a per-head product writes).
//
// Rotation: pair i is dims (2i, 2i + 1) of the rotated part (interleaved) or (i, i + n/2)
// (half-split), over its first rot_dims dims; the rest passes unchanged.
#include "common.h"
#include "mercury_kernels.h"

__device__ __forceinline__ float weight_at(const void* w, int bf16, int i) {
  return bf16 ? bf16_to_f32(((const bf16_t*)w)[i]) : ((const float*)w)[i];
}

// One of the pair's members after the turn: j within the rotated part.
__device__ __forceinline__ float turned(const float* x, int j, int rot_dims, int interleaved,
                                        const float* cs, const float* sn) {
  if (j >= rot_dims) return x[j];
  const int half = rot_dims / 2;
  if (interleaved) {
    const int pair = j >> 1;
    return (j & 1) ? x[j] * cs[pair] + x[j - 1] * sn[pair] : x[j] * cs[pair] - x[j + 1] * sn[pair];
  }
  return j < half ? x[j] * cs[j] - x[j + half] * sn[j]
                  : x[j] * cs[j - half] + x[j - half] * sn[j - half];
}

template <typename T>
__global__ void latent_prepare_kernel(const float* __restrict__ down, int down_stride, int q_rank,
                                      int kv_rank, int rot, const void* __restrict__ q_norm_w,
                                      const void* __restrict__ kv_norm_w, int norm_bf16, float eps,
                                      const float* __restrict__ cos_table,
                                      const float* __restrict__ sin_table, int rot_dims,
                                      int interleaved, const int* __restrict__ positions,
                                      const int* __restrict__ token_seq,
                                      const int* __restrict__ block_table, int table_stride,
                                      T* __restrict__ q_latent, T* __restrict__ k_cache,
                                      T* __restrict__ v_cache, int page_shift, int write_kv,
                                      int key_width, int value_width) {
  __shared__ float scratch[16];
  extern __shared__ float rotated[];     // the token's raw rotated key part
  const int t = blockIdx.x;
  const float* row = down + (size_t)t * down_stride;
  if (q_rank > 0) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) sq = fmaf(row[i], row[i], sq);
    const float rstd = 1.f / sqrtf(block_sum(sq, scratch) / (float)q_rank + eps);
    T* dst = q_latent + (size_t)t * q_rank;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
      Elem<T>::store(dst + i, row[i] * rstd * weight_at(q_norm_w, norm_bf16, i));
  }
  if (!write_kv) return;
  const int pos = positions[t];
  const int page_size = 1 << page_shift;
  const int page = block_table[(size_t)token_seq[t] * table_stride + (pos >> page_shift)];
  if (page < 0) return;  // the host never schedules a write into a page that was given back
  const int off = pos & (page_size - 1);
  const float* c = row + q_rank;
  float sq = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) sq = fmaf(c[i], c[i], sq);
  const float rstd = 1.f / sqrtf(block_sum(sq, scratch) / (float)kv_rank + eps);
  // rows of key_width >= kv_rank + rot and value_width >= kv_rank: what lies beyond is zero
  T* k_dst = k_cache + ((size_t)page * page_size + off) * key_width;
  T* v_dst = v_cache + (size_t)page * value_width * page_size + off;
  for (int i = kv_rank + rot + threadIdx.x; i < key_width; i += blockDim.x) Elem<T>::store(k_dst + i, 0.f);
  for (int i = kv_rank + threadIdx.x; i < value_width; i += blockDim.x)
    Elem<T>::store(v_dst + (size_t)i * page_size, 0.f);
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const float v = c[i] * rstd * weight_at(kv_norm_w, norm_bf16, i);
    Elem<T>::store(k_dst + i, v);
    Elem<T>::store(v_dst + (size_t)i * page_size, v);
  }
  for (int i = threadIdx.x; i < rot; i += blockDim.x) rotated[i] = c[kv_rank + i];
  __syncthreads();
  const float* cs = cos_table + (size_t)pos * (rot_dims / 2);
  const float* sn = sin_table + (size_t)pos * (rot_dims / 2);
  for (int i = threadIdx.x; i < rot; i += blockDim.x)
    Elem<T>::store(k_dst + kv_rank + i, turned(rotated, i, rot_dims, interleaved, cs, sn));
}

extern "C" int mk_latent_prepare(const float* down, int down_stride, int q_rank, int kv_rank,
                                 int rot, const void* q_norm_w, const void* kv_norm_w,
                                 int norm_dtype, float eps, const float* cos_table,
                                 const float* sin_table, int table_positions, int rot_dims,
                                 int interleaved, const int* positions, const int* token_seq,
                                 const int* block_table, int table_stride, void* q_latent,
                                 void* k_cache, void* v_cache, int key_width, int value_width,
                                 int dtype, int page_size, int write_kv, int tokens,
                                 hipStream_t stream) {
  MK_REQUIRE(!write_kv || (key_width >= kv_rank + rot && value_width >= kv_rank),
             "latent_prepare: cache rows of %d / %d are too narrow", key_width, value_width);
  MK_REQUIRE(tokens >= 0 && q_rank >= 0 && kv_rank > 0 && rot >= 0, "latent_prepare: bad sizes");
  MK_REQUIRE(down_stride >= q_rank + (write_kv ? kv_rank + rot : 0),
             "latent_prepare: rows of %d hold no [%d | %d | %d]", down_stride, q_rank, kv_rank, rot);
  MK_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0,
             "latent_prepare: %d rotated dims of %d", rot_dims, rot);
  MK_REQUIRE(rot_dims == 0 || (cos_table && sin_table && table_positions > 0),
             "latent_prepare: no angle tables");
  MK_REQUIRE(mk_is_pow2(page_size), "latent_prepare: page size %d is not a power of two", page_size);
  MK_REQUIRE(norm_dtype == MK_F32 || norm_dtype == MK_BF16, "latent_prepare: norm dtype %d", norm_dtype);
  MK_REQUIRE(rot * 4 <= 48 * 1024, "latent_prepare: rotated part of %d is too wide", rot);
  MK_REQUIRE(q_rank == 0 || q_latent, "latent_prepare: no room for the query latent");
  MK_REQUIRE(!write_kv || (k_cache && v_cache), "latent_prepare: no cache to write");
  if (tokens == 0) return 0;
  const int widest = q_rank > kv_rank ? q_rank : kv_rank;
  const int threads = widest >= 256 ? 256 : (widest + 63) / 64 * 64;
  const size_t lds = (size_t)(rot > 0 ? rot : 1) * 4;
#define LP_LAUNCH(T)                                                                              \
  latent_prepare_kernel<T><<<tokens, threads, lds, stream>>>(                                     \
      down, down_stride, q_rank, kv_rank, rot, q_norm_w, kv_norm_w, norm_dtype == MK_BF16, eps,   \
      cos_table, sin_table, rot_dims, interleaved, positions, token_seq, block_table,             \
      table_stride, (T*)q_latent, (T*)k_cache, (T*)v_cache, mk_log2(page_size), write_kv,         \
      key_width, value_width)
  if (dtype == MK_F32) LP_LAUNCH(float);
  else if (dtype == MK_BF16) LP_LAUNCH(bf16_t);
  else MK_REQUIRE(false, "latent_prepare: unknown dtype %d", dtype);
#undef LP_LAUNCH
  MK_LAUNCH_CHECK("latent_prepare");
  return 0;
}

// q [T, heads, dim + rot] -> out [T, heads, out_width]: the rotated part of each head, turned
// by the token's position, lands at out[t, head, out_offset ..].
template <typename T>
__global__ void latent_query_tail_kernel(const T* __restrict__ q, int heads, int dim, int rot,
                                         const float* __restrict__ cos_table,
                                         const float* __restrict__ sin_table, int rot_dims,
                                         int interleaved, const int* __restrict__ positions,
                                         T* __restrict__ out, int out_width, int out_offset) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const float* cs = cos_table + (size_t)pos * (rot_dims / 2);
  const float* sn = sin_table + (size_t)pos * (rot_dims / 2);
  const T* row = q + (size_t)t * heads * (dim + rot);
  for (int idx = threadIdx.x; idx < heads * rot; idx += blockDim.x) {
    const int head = idx / rot, j = idx - head * rot;
    const T* x = row + head * (dim + rot) + dim;
    float y = Elem<T>::load(x + j);
    if (j < rot_dims) {
      const int half = rot_dims / 2;
      if (interleaved) {
        const int pair = j >> 1;
        y = (j & 1) ? y * cs[pair] + Elem<T>::load(x + j - 1) * sn[pair]
                    : y * cs[pair] - Elem<T>::load(x + j + 1) * sn[pair];
      } else {
        y = j < half ? y * cs[j] - Elem<T>::load(x + j + half) * sn[j]
                     : y * cs[j - half] + Elem<T>::load(x + j - half) * sn[j - half];
      }
    }
    Elem<T>::store(out + ((size_t)t * heads + head) * out_width + out_offset + j, y);
  }
  // what lies behind the rotated part in a row of the output is zero
  const int pad = out_width - out_offset - rot;
  for (int idx = threadIdx.x; idx < heads * pad; idx += blockDim.x) {
    const int head = idx / pad, j = idx - head * pad;
    Elem<T>::store(out + ((size_t)t * heads + head) * out_width + out_offset + rot + j, 0.f);
  }
}

extern "C" int mk_latent_query_tail(const void* q, int dtype, int heads, int dim, int rot,
                                    const float* cos_table, const float* sin_table,
                                    int table_positions, int rot_dims, int interleaved,
                                    const int* positions, void* out, int out_width, int out_offset,
                                    int tokens, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && heads > 0 && dim >= 0 && rot >= 0, "latent_query_tail: bad sizes");
  MK_REQUIRE(out_offset >= 0 && out_offset + rot <= out_width, "latent_query_tail: no room");
  MK_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0,
             "latent_query_tail: %d rotated dims of %d", rot_dims, rot);
  MK_REQUIRE(rot_dims == 0 || (cos_table && sin_table && table_positions > 0),
             "latent_query_tail: no angle tables");
  if (tokens == 0 || out_offset == out_width) return 0;
  const int work = heads * (out_width - out_offset);
  const int threads = work >= 256 ? 256 : (work + 63) / 64 * 64;
  if (dtype == MK_F32)
    latent_query_tail_kernel<float><<<tokens, threads, 0, stream>>>(
        (const float*)q, heads, dim, rot, cos_table, sin_table, rot_dims, interleaved, positions,
        (float*)out, out_width, out_offset);
  else if (dtype == MK_BF16)
    latent_query_tail_kernel<bf16_t><<<tokens, threads, 0, stream>>>(
        (const bf16_t*)q, heads, dim, rot, cos_table, sin_table, rot_dims, interleaved, positions,
        (bf16_t*)out, out_width, out_offset);
  else
    MK_REQUIRE(false, "latent_query_tail: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("latent_query_tail");
  return 0;
}
