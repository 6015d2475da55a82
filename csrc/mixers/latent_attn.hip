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

// ---------------------------------------------------------------------------------
// Split-key kernel for decode rows and short segments.  A workgroup owns (one query
// row, one slice of its keys, one group of up to 16 heads): it stages tiles of cache
// rows in LDS (coalesced, widened to fp32, odd row stride against bank conflicts) and
// every head of the group scores and accumulates against the same tile, so a cache row
// is read once per head group instead of once per head.  Each workgroup leaves (max,
// sum, weighted c sums) per head; latent_combine_kernel merges the slices.
// ---------------------------------------------------------------------------------
// sum over the 16 lanes of a row (quad swaps, mirrored half row, mirrored row): every
// lane gets the total
__device__ __forceinline__ float sum16(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));
  return v;
}

constexpr int kSplitTK = 8;    // keys per staged tile (compile time: the inner loops carry no branches)

// Stages cnt <= kSplitTK cache rows (keys k0..) into LDS as fp32, a wave per key: the wave's
// keys' block-table entries and all their 16-byte loads are issued before anything is
// stored, so one memory latency covers the tile.  Rows narrower than 16-byte groups, or
// wider than 4 groups per lane, take the element-wise path.
template <typename TC>
__device__ __forceinline__ void stage_tile(float* __restrict__ kt, int ldk, const TC* __restrict__ cache,
                                           const int* __restrict__ tab, int k0, int cnt, int width,
                                           int block_size, int num_blocks, int wv, int lane) {
  constexpr int VE = 16 / (int)sizeof(TC);          // elements per 16-byte group
  constexpr int KW = kSplitTK / 4, CH = 4;          // keys per wave, groups per lane and key
  // rows past the tile's last key read as zeros (their scores are masked afterwards)
#pragma unroll
  for (int u = 0; u < KW; ++u)
    if (wv + 4 * u >= cnt)
      for (int i = lane; i < width; i += 64) kt[(wv + 4 * u) * ldk + i] = 0.f;
  const int groups = width / VE;
  long base[KW];
#pragma unroll
  for (int u = 0; u < KW; ++u) {
    const int j = wv + 4 * u;
    base[u] = -1;
    if (j < cnt) {
      const int tok = k0 + j;
      int blk = tab[tok / block_size];
      if (blk < 0 || blk >= num_blocks) blk = 0;
      base[u] = ((long)blk * block_size + tok % block_size) * width;
    }
  }
  if (width % VE == 0 && groups <= 64 * CH) {
    uint4 v[KW][CH];
#pragma unroll
    for (int u = 0; u < KW; ++u)
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int gidx = lane + 64 * c;
        if (base[u] >= 0 && gidx < groups)
          v[u][c] = *reinterpret_cast<const uint4*>(cache + base[u] + (long)gidx * VE);
      }
#pragma unroll
    for (int u = 0; u < KW; ++u)
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int gidx = lane + 64 * c;
        if (base[u] >= 0 && gidx < groups) {
          float* dst = kt + (wv + 4 * u) * ldk + gidx * VE;
          if constexpr (sizeof(TC) == 2) {
            float f[8];
            ft::load8(v[u][c], f);
#pragma unroll
            for (int k = 0; k < 8; ++k) dst[k] = f[k];
          } else {
            dst[0] = __uint_as_float(v[u][c].x);
            dst[1] = __uint_as_float(v[u][c].y);
            dst[2] = __uint_as_float(v[u][c].z);
            dst[3] = __uint_as_float(v[u][c].w);
          }
        }
      }
  } else {
#pragma unroll
    for (int u = 0; u < KW; ++u)
      if (base[u] >= 0)
        for (int i = lane; i < width; i += 64) kt[(wv + 4 * u) * ldk + i] = ld(cache, base[u] + i);
  }
}


// 256 threads = 16 heads x 16 lanes.  The 16 lanes of a head split the dot products'
// dimension (scores) and the rank axis (sums); scores are reduced over them on the lane
// permute path, the softmax state (running max / sum) and the sums live in registers,
// so the only barriers are those around staging a tile.  ACC = ceil(rank / 16).
template <typename TC, int ACC>
__global__ void __launch_bounds__(256)
latent_split_kernel(float* __restrict__ ws_acc, float* __restrict__ ws_ml, const float* __restrict__ qa,
                    const float* __restrict__ qr, const TC* __restrict__ cache, const int* __restrict__ start,
                    const int* __restrict__ pos0, const int* __restrict__ kv_len, const int* __restrict__ bt,
                    int bt_stride, int heads, long total_rows, int rank, int dr, int block_size,
                    int num_blocks, float scale, int skip_from, int splits, int hg, int tk) {
  extern __shared__ float smem[];
  const int s = blockIdx.z;
  const int r0 = start[s], n = start[s + 1] - r0;
  const int rel = blockIdx.y;
  if (rel >= n || (skip_from > 0 && n >= skip_from)) return;
  const long row = r0 + rel;
  const int sp = blockIdx.x % splits, h0 = (blockIdx.x / splits) * hg;
  const int nh = min(hg, heads - h0);
  const int width = rank + dr, ldk = width | 1;   // odd strides: heads / keys land on different banks
  float* qs = smem;                       // [hg, ldk]
  float* kt = qs + hg * ldk;              // [tk, ldk]
  const int tid = threadIdx.x;
  const int hl = tid >> 4, ds = tid & 15;
  const bool on = hl < nh;
  int nk = pos0[s] + rel + 1;
  if (nk > kv_len[s]) nk = kv_len[s];
  const int per = (nk + splits - 1) / splits;
  const int chunk = (per + tk - 1) / tk * tk;
  const int k_begin = sp * chunk, k_end = min(nk, k_begin + chunk);
  const int* tab = bt + (long)s * bt_stride;
  const int wv = tid >> 6, lane = tid & 63;
  for (int h = wv; h < nh; h += 4) {      // a wave per head: independent coalesced loads
    const float* qah = qa + ((long)(h0 + h) * total_rows + row) * rank;
    const float* qrh = qr + (row * heads + h0 + h) * dr;
    for (int i = lane; i < rank; i += 64) qs[h * ldk + i] = qah[i];
    for (int i = lane; i < dr; i += 64) qs[h * ldk + rank + i] = qrh[i];
  }
  float m = -INFINITY, l = 0.f;
  float acc[ACC];
#pragma unroll
  for (int a = 0; a < ACC; ++a) acc[a] = 0.f;
  const float* q = qs + (on ? hl : 0) * ldk;
  for (int k0 = k_begin; k0 < k_end; k0 += tk) {
    const int cnt = min(tk, k_end - k0);
    __syncthreads();                      // the previous tile is no longer read
    stage_tile<TC>(kt, ldk, cache, tab, k0, cnt, width, block_size, num_blocks, wv, lane);
    __syncthreads();
    float p[kSplitTK];
#pragma unroll
    for (int j = 0; j < kSplitTK; ++j) p[j] = 0.f;
    for (int i = ds; i < width; i += 16) {
      const float qv = q[i];
#pragma unroll
      for (int j = 0; j < kSplitTK; ++j) p[j] += qv * kt[j * ldk + i];
    }
    float mt = -INFINITY;
#pragma unroll
    for (int j = 0; j < kSplitTK; ++j) {
      p[j] = j < cnt ? sum16(p[j]) * scale : -INFINITY;   // (the select follows the reduction)
      mt = fmaxf(mt, p[j]);
    }
    const float mn = fmaxf(m, mt);
    const float alpha = expf(m - mn);     // 0 at the first tile (m = -inf)
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < kSplitTK; ++j) {
      p[j] = expf(p[j] - mn);             // exp(-inf) = 0 for the masked keys
      sum += p[j];
    }
    l = l * alpha + sum;
    m = mn;
#pragma unroll
    for (int a = 0; a < ACC; ++a) {
      const int d = ds + 16 * a;
      float v = acc[a] * alpha;
      if (d < rank) {
#pragma unroll
        for (int j = 0; j < kSplitTK; ++j) v += p[j] * kt[j * ldk + d];
      }
      acc[a] = v;
    }
  }
  if (on) {
    const long base = (row * splits + sp) * heads + h0 + hl;
#pragma unroll
    for (int a = 0; a < ACC; ++a) {
      const int d = ds + 16 * a;
      if (d < rank) ws_acc[base * rank + d] = acc[a];
    }
    if (ds == 0) {
      ws_ml[base * 2] = m;
      ws_ml[base * 2 + 1] = l;
    }
  }
}

// out[h, row, :] = sum_s exp(m_s - M) acc_s / sum_s exp(m_s - M) l_s over the key slices
__global__ void latent_combine_kernel(float* __restrict__ out, const float* __restrict__ ws_acc,
                                      const float* __restrict__ ws_ml, const int* __restrict__ start,
                                      int heads, long total_rows, int rank, int skip_from, int splits) {
  const int s = blockIdx.y;
  const int r0 = start[s], n = start[s + 1] - r0;
  const int rel = blockIdx.x;
  if (rel >= n || (skip_from > 0 && n >= skip_from)) return;
  const long row = r0 + rel;
  const int h = blockIdx.z;
  float M = -INFINITY;
  for (int sp = 0; sp < splits; ++sp) M = fmaxf(M, ws_ml[((row * splits + sp) * heads + h) * 2]);
  float L = 0.f;
  for (int sp = 0; sp < splits; ++sp) {
    const long b = (row * splits + sp) * heads + h;
    const float m = ws_ml[b * 2];
    L += m == -INFINITY ? 0.f : expf(m - M) * ws_ml[b * 2 + 1];
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    float v = 0.f;
    for (int sp = 0; sp < splits; ++sp) {
      const long b = (row * splits + sp) * heads + h;
      const float m = ws_ml[b * 2];
      const float w = m == -INFINITY ? 0.f : expf(m - M);   // an empty slice left zeros
      v += w * ws_acc[b * rank + d];
    }
    out[((long)h * total_rows + row) * rank + d] = v * inv;
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

// plan of the split-key kernel for these sizes: heads per group, keys per tile, LDS
// bytes, accumulators per thread (0: does not fit, use the per-row kernel)
static int split_plan(int heads, int rank, int dr, int* hg, int* tk, size_t* lds) {
  const int width = rank + dr, ldk = width | 1;
  int g = heads < 16 ? heads : 16;
  const long budget = 64 * 1024 / 4 - 64;
  while (g > 1 && (long)(g + kSplitTK) * ldk > budget) --g;
  if ((long)(g + kSplitTK) * ldk > budget) return 0;
  const int acc = (rank + 15) / 16;
  if (acc > 64) return 0;
  *hg = g;
  *tk = kSplitTK;
  *lds = (size_t)(g + kSplitTK) * ldk * sizeof(float);
  return acc;
}

extern "C" long mx_latent_split_ws(int heads, int rank, int dr) {
  int hg, tk;
  size_t lds;
  return split_plan(heads, rank, dr, &hg, &tk, &lds) ? 1 : 0;
}

template <typename TC, int ACC>
static void launch_split(dim3 grid, size_t lds, hipStream_t s, float* ws_acc, float* ws_ml, const float* qa,
                         const float* qr, const void* cache, const int* start, const int* pos0,
                         const int* kv_len, const int* bt, int bt_stride, int heads, long total_rows, int rank,
                         int dr, int block_size, int num_blocks, float scale, int skip_from, int splits, int hg,
                         int tk) {
  hipLaunchKernelGGL((latent_split_kernel<TC, ACC>), grid, dim3(256), lds, s, ws_acc, ws_ml, qa, qr,
                     (const TC*)cache, start, pos0, kv_len, bt, bt_stride, heads, total_rows, rank, dr,
                     block_size, num_blocks, scale, skip_from, splits, hg, tk);
}

extern "C" int mx_latent_attention_split(float* out, float* ws_acc, float* ws_ml, const float* qa,
                                         const float* qr, const void* cache, int cache_bf16, const int* start,
                                         const int* pos0, const int* kv_len, const int* bt, int bt_stride,
                                         int num_segs, int max_rows, int heads, long total_rows, int rank,
                                         int dr, int block_size, int num_blocks, float scale, int skip_from,
                                         int splits, hipStream_t s) {
  if (num_segs <= 0 || max_rows <= 0) return 0;
  if (skip_from > 0 && max_rows >= skip_from) max_rows = skip_from - 1;
  if (max_rows <= 0) return 0;
  int hg, tk;
  size_t lds;
  const int acc = split_plan(heads, rank, dr, &hg, &tk, &lds);
  if (!acc || splits < 1 || max_rows > 65535 || num_segs > 65535 || heads > 65535) return -1;
  const int groups = (heads + hg - 1) / hg;
  const dim3 grid(splits * groups, max_rows, num_segs);
#define MX_SPLIT(A)                                                                                      \
  do {                                                                                                   \
    if (cache_bf16)                                                                                      \
      launch_split<bf16_t, A>(grid, lds, s, ws_acc, ws_ml, qa, qr, cache, start, pos0, kv_len, bt,       \
                              bt_stride, heads, total_rows, rank, dr, block_size, num_blocks, scale,     \
                              skip_from, splits, hg, tk);                                                \
    else                                                                                                 \
      launch_split<float, A>(grid, lds, s, ws_acc, ws_ml, qa, qr, cache, start, pos0, kv_len, bt,        \
                             bt_stride, heads, total_rows, rank, dr, block_size, num_blocks, scale,      \
                             skip_from, splits, hg, tk);                                                 \
  } while (0)
  if (acc <= 4) MX_SPLIT(4);
  else if (acc <= 8) MX_SPLIT(8);
  else if (acc <= 16) MX_SPLIT(16);
  else if (acc <= 32) MX_SPLIT(32);
  else MX_SPLIT(64);
#undef MX_SPLIT
  hipLaunchKernelGGL(latent_combine_kernel, dim3(max_rows, num_segs, heads), dim3(rank >= 256 ? 256 : 64), 0,
                     s, out, ws_acc, ws_ml, start, heads, total_rows, rank, skip_from, splits);
  return (int)hipGetLastError();
}
