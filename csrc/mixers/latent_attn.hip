// Latent attention over a paged cache whose rows are [c (rank) | rotated shared key (dr)]:
//   * latent_kv_write: c = rms_norm(down-projection[:rank]) * w, key part rotated
//     (rotate-half pairs over its first `dims` entries, fp32 angles from a table),
//   * latent_q_rope: splits query rows into unrotated and rotated fp32 parts,
//   * latent_attention: causal softmax of (qa . c + qr . k_rot) * scale over the paged
//     rows, returning the weighted sums of the c parts (the value up-projection is
//     applied by the caller), fp32 scores / weights / sums.
//
// The attention kernel runs one workgroup per query row; its waves take the heads in
// turn.  A wave scores 64 keys at a time (one key per lane), keeps a running max / sum
// (online softmax) and accumulates the weighted c rows with the rank axis spread over
// the lanes.  Rows of a segment at position p see keys 0..p.
#include "mx_common.h"

namespace mx {

template <typename T, typename TC, int NT>
__global__ void latent_kv_write_kernel(const T* __restrict__ dkv, long stride, const float* __restrict__ w,
                                       float eps, const float* __restrict__ table, int table_rows,
                                       int dims, const int* __restrict__ positions,
                                       const int* __restrict__ slots, TC* __restrict__ cache, long num_slots,
                                       int rank, int dr) {
  __shared__ float red[NT / 64];
  const long row = blockIdx.x;
  const long sl = slots[row];
  if (sl < 0 || sl >= num_slots) return;
  const T* x = dkv + row * stride;
  TC* dst = cache + sl * (rank + dr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += NT) {
    const float v = ld(x, i);
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)rank + eps);
  for (int i = threadIdx.x; i < rank; i += NT) st(dst, i, ld(x, i) * r * w[i]);
  int p = positions[row];
  p = p < 0 ? 0 : (p >= table_rows ? table_rows - 1 : p);
  const float* cs = table + (long)p * dims;
  const int half = dims / 2;
  for (int i = threadIdx.x; i < dr; i += NT) {
    float v;
    if (i < half) v = ld(x, rank + i) * cs[i] - ld(x, rank + i + half) * cs[half + i];
    else if (i < dims) v = ld(x, rank + i) * cs[i - half] + ld(x, rank + i - half) * cs[i];
    else v = ld(x, rank + i);
    st(dst, rank + i, v);
  }
}

template <typename T>
__global__ void latent_q_rope_kernel(float* __restrict__ qn, float* __restrict__ qr,
                                     const T* __restrict__ q, long stride, const float* __restrict__ table,
                                     int table_rows, int dims, const int* __restrict__ positions, int heads,
                                     int dn, int dr) {
  const long row = blockIdx.x;
  int p = positions[row];
  p = p < 0 ? 0 : (p >= table_rows ? table_rows - 1 : p);
  const float* cs = table + (long)p * dims;
  const int half = dims / 2, hd = dn + dr;
  const T* x = q + row * stride;
  for (int e = threadIdx.x; e < heads * hd; e += blockDim.x) {
    const int h = e / hd, i = e % hd;
    if (i < dn) {
      qn[(row * heads + h) * dn + i] = ld(x, e);
    } else {
      const int j = i - dn;
      float v;
      if (j < half) v = ld(x, e) * cs[j] - ld(x, e + half) * cs[half + j];
      else if (j < dims) v = ld(x, e) * cs[j - half] + ld(x, e - half) * cs[j];
      else v = ld(x, e);
      qr[(row * heads + h) * dr + j] = v;
    }
  }
}

// grid (max_rows, segments); RPL = latent entries per lane (rank <= 64 RPL)
template <typename TC, int RPL>
__global__ void __launch_bounds__(256)
latent_attention_kernel(float* __restrict__ out, const float* __restrict__ qa, const float* __restrict__ qr,
                        const TC* __restrict__ cache, const int* __restrict__ start,
                        const int* __restrict__ pos0, const int* __restrict__ kv_len,
                        const int* __restrict__ bt, int bt_stride, int heads, long total_rows, int rank,
                        int dr, int block_size, int num_blocks, float scale, int skip_from) {
  extern __shared__ float smem[];
  const int s = blockIdx.y;
  const int r0 = start[s], n = start[s + 1] - r0;
  const int rel = blockIdx.x;
  if (rel >= n || (skip_from > 0 && n >= skip_from)) return;   // long segments: the product path
  const long row = r0 + rel;
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const int width = rank + dr;
  float* qs = smem + (long)wid * width;          // this wave's query
  int nk = pos0[s] + rel + 1;                    // causal: keys 0 .. position
  if (nk > kv_len[s]) nk = kv_len[s];
  const int* tab = bt + (long)s * bt_stride;
  for (int h = wid; h < heads; h += nw) {
    const float* qah = qa + ((long)h * total_rows + row) * rank;
    const float* qrh = qr + (row * heads + h) * dr;
    __builtin_amdgcn_wave_barrier();   // the previous head's reads of qs come first
    for (int i = lane; i < rank; i += 64) qs[i] = qah[i];
    for (int i = lane; i < dr; i += 64) qs[rank + i] = qrh[i];
    // a wave's LDS writes are visible to its own later reads in program order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    float m = -INFINITY, l = 0.f;
    float acc[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) acc[r] = 0.f;
    for (int k0 = 0; k0 < nk; k0 += 64) {
      const int j = k0 + lane;
      float sc = -INFINITY;
      long base = 0;
      if (j < nk) {
        int blk = tab[j / block_size];
        if (blk < 0 || blk >= num_blocks) blk = 0;
        base = ((long)blk * block_size + j % block_size) * width;
        float d = 0.f;
        for (int i = 0; i < width; ++i) d += qs[i] * ld(cache, base + i);
        sc = d * scale;
      }
      const float mt = ft::wave_max(sc);
      const float mn = fmaxf(m, mt);
      const float alpha = expf(m - mn);          // m = -inf at the first tile: alpha = 0
      const float p = j < nk ? expf(sc - mn) : 0.f;
      l = l * alpha + ft::wave_sum(p);
      m = mn;
#pragma unroll
      for (int r = 0; r < RPL; ++r) acc[r] *= alpha;
      const int cnt = nk - k0 < 64 ? nk - k0 : 64;
      for (int jj = 0; jj < cnt; ++jj) {
        const float pj = __shfl(p, jj, 64);
        const long bj = __shfl(base, jj, 64);
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
          const int i = lane + 64 * r;
          if (i < rank) acc[r] += pj * ld(cache, bj + i);
        }
      }
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    float* op = out + ((long)h * total_rows + row) * rank;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int i = lane + 64 * r;
      if (i < rank) op[i] = acc[r] * inv;
    }
  }
}

// P[r, j] = softmax_j(scale * S[r, j]) over the keys j <= first_pos + (r mod rows_per_head),
// 0 beyond (rows r = head * rows_per_head + query row); fp32 statistics, P in TP
template <typename TP, int NT>
__global__ void causal_softmax_kernel(TP* __restrict__ P, const float* __restrict__ S, int rows_per_head,
                                      int first_pos, int ncols, float scale) {
  __shared__ float red[NT / 64];
  __shared__ float bmax;
  const long r = blockIdx.x;
  const int valid = min(first_pos + (int)(r % rows_per_head) + 1, ncols);
  const float* sr = S + r * ncols;
  float m = -INFINITY;
  for (int j = threadIdx.x; j < valid; j += NT) m = fmaxf(m, sr[j] * scale);
  m = ft::wave_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float b = red[0];
    for (int w = 1; w < NT / 64; ++w) b = fmaxf(b, red[w]);
    bmax = b;
  }
  __syncthreads();
  m = bmax;
  float sum = 0.f;
  for (int j = threadIdx.x; j < valid; j += NT) sum += expf(sr[j] * scale - m);
  sum = block_sum<NT>(sum, red);
  const float inv = sum > 0.f ? 1.0f / sum : 0.f;
  for (int j = threadIdx.x; j < ncols; j += NT)
    st(P, r * ncols + j, j < valid ? expf(sr[j] * scale - m) * inv : 0.f);
}

}  // namespace mx

using namespace mx;

extern "C" int mx_causal_softmax(void* P, int p_bf16, const float* S, long rows, int rows_per_head,
                                 int first_pos, int ncols, float scale, hipStream_t s) {
  if (rows <= 0 || ncols <= 0) return 0;
  if (p_bf16)
    hipLaunchKernelGGL((causal_softmax_kernel<bf16_t, 256>), dim3((unsigned)rows), dim3(256), 0, s, (bf16_t*)P, S,
                       rows_per_head, first_pos, ncols, scale);
  else
    hipLaunchKernelGGL((causal_softmax_kernel<float, 256>), dim3((unsigned)rows), dim3(256), 0, s, (float*)P, S,
                       rows_per_head, first_pos, ncols, scale);
  return (int)hipGetLastError();
}

extern "C" int mx_latent_kv_write(const void* dkv, int bf16, long stride, const float* w, float eps,
                                  const float* table, int table_rows, int dims, const int* positions,
                                  const int* slots, void* cache, int cache_bf16, long num_slots, long rows,
                                  int rank, int dr, hipStream_t s) {
  if (rows <= 0) return 0;
  const dim3 grid((unsigned)rows), block(256);
  if (bf16 && cache_bf16)
    hipLaunchKernelGGL((latent_kv_write_kernel<bf16_t, bf16_t, 256>), grid, block, 0, s, (const bf16_t*)dkv,
                       stride, w, eps, table, table_rows, dims, positions, slots, (bf16_t*)cache, num_slots,
                       rank, dr);
  else if (!bf16 && !cache_bf16)
    hipLaunchKernelGGL((latent_kv_write_kernel<float, float, 256>), grid, block, 0, s, (const float*)dkv,
                       stride, w, eps, table, table_rows, dims, positions, slots, (float*)cache, num_slots,
                       rank, dr);
  else
    return -1;
  return (int)hipGetLastError();
}

extern "C" int mx_latent_q_rope(float* qn, float* qr, const void* q, int bf16, long stride,
                                const float* table, int table_rows, int dims, const int* positions,
                                long rows, int heads, int dn, int dr, hipStream_t s) {
  if (rows <= 0) return 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((latent_q_rope_kernel<T>), dim3((unsigned)rows), dim3(256), 0, s,
                                         qn, qr, (const T*)q, stride, table, table_rows, dims, positions,
                                         heads, dn, dr));
  return (int)hipGetLastError();
}

extern "C" int mx_latent_max_rank() { return 64 * 16; }

template <typename TC, int RPL>
static void launch_latent(dim3 grid, size_t lds, hipStream_t s, float* out, const float* qa, const float* qr,
                          const void* cache, const int* start, const int* pos0, const int* kv_len,
                          const int* bt, int bt_stride, int heads, long total_rows, int rank, int dr,
                          int block_size, int num_blocks, float scale, int skip_from) {
  hipLaunchKernelGGL((latent_attention_kernel<TC, RPL>), grid, dim3(256), lds, s, out, qa, qr,
                     (const TC*)cache, start, pos0, kv_len, bt, bt_stride, heads, total_rows, rank, dr,
                     block_size, num_blocks, scale, skip_from);
}

extern "C" int mx_latent_attention(float* out, const float* qa, const float* qr, const void* cache,
                                   int cache_bf16, const int* start, const int* pos0, const int* kv_len,
                                   const int* bt, int bt_stride, int num_segs, int max_rows, int heads,
                                   long total_rows, int rank, int dr, int block_size, int num_blocks,
                                   float scale, int skip_from, hipStream_t s) {
  if (num_segs <= 0 || max_rows <= 0) return 0;
  if (rank < 1 || rank > mx_latent_max_rank() || max_rows > 65535 * 32 || num_segs > 65535) return -1;
  const size_t lds = (size_t)4 * (rank + dr) * sizeof(float);
  if (lds > 60 * 1024) return -2;
  if (skip_from > 0 && max_rows >= skip_from) max_rows = skip_from - 1;
  if (max_rows <= 0) return 0;
  const dim3 grid(max_rows, num_segs);
  const int need = (rank + 63) / 64;
#define MX_LAT(RPL)                                                                                     \
  do {                                                                                                  \
    if (cache_bf16)                                                                                     \
      launch_latent<bf16_t, RPL>(grid, lds, s, out, qa, qr, cache, start, pos0, kv_len, bt, bt_stride,  \
                                 heads, total_rows, rank, dr, block_size, num_blocks, scale, skip_from); \
    else                                                                                                \
      launch_latent<float, RPL>(grid, lds, s, out, qa, qr, cache, start, pos0, kv_len, bt, bt_stride,   \
                                heads, total_rows, rank, dr, block_size, num_blocks, scale, skip_from); \
  } while (0)
  if (need <= 1) MX_LAT(1);
  else if (need <= 2) MX_LAT(2);
  else if (need <= 4) MX_LAT(4);
  else if (need <= 8) MX_LAT(8);
  else MX_LAT(16);
#undef MX_LAT
  return (int)hipGetLastError();
}
