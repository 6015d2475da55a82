// Selective state-space scan with one scalar decay per head and row over fp32 state
// slots, and the gated grouped RMS norm that follows it.
//
// Rows come in segments as in delta_rule.hip (start / pos0 / slot; a segment at
// position 0 starts from zeros; slot < 0 is padding).  Rows of xbc are
// [x (heads*dv) | B (groups*n) | C (groups*n)].  Per head h (group h / (heads/groups)):
//   step = softplus(dt + dt_bias[h]);  decay = exp(-exp(a_log[h]) * step)
//   S <- decay S + step B x^T   (S is n x dv);   y = S^T C + d_skip[h] x
// Columns of S are independent, so a workgroup owns 32 columns of one head of one
// sequence: 8 lanes share a column, each holding n/8 state rows in registers, the
// output dot product reduced over those 8 lanes; a segment's rows are walked in order
// with the per-row inputs staged through LDS in double-buffered chunks.
#include "mx_common.h"

namespace mx {

constexpr int kSL = 8;         // lanes that share one state column
constexpr int kSCols = 32;     // state columns per workgroup (256 threads)

__device__ __forceinline__ float ssd_sum8(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // lanes ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // lanes ^ 2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // 7 - lane
  return v;
}

template <int R>
struct SsdTile {
  static constexpr int TT = R <= 16 ? 16 : 8;                 // rows per chunk
  static constexpr int NP = 8 * R;                            // padded state size
  static constexpr int ROWF = 2 * NP + kSCols + 2;            // floats per staged row: B | C | x | step | decay
  static constexpr int NLD = (TT * 2 * NP + 255) / 256;       // B/C loads per thread and chunk
  static constexpr int NV = (TT * kSCols + 255) / 256;        // x loads per thread and chunk
};

template <typename T, int R>
__global__ void __launch_bounds__(256)
ssd_scan_kernel(float* __restrict__ y, const T* __restrict__ xbc, long x_stride, const T* __restrict__ dt,
                long dt_stride, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                const float* __restrict__ d_skip, float* __restrict__ state, const int* __restrict__ start,
                const int* __restrict__ pos0, const int* __restrict__ slot, int heads, int groups, int n,
                int dv, int num_slots) {
  using P = SsdTile<R>;
  __shared__ float stage[2][P::TT * P::ROWF];
  const int s = blockIdx.z, h = blockIdx.y;
  const int sl = slot[s];
  const int r0 = start[s], rows = start[s + 1] - r0;
  const int tid = threadIdx.x;
  const int kl = tid & (kSL - 1);
  const int cl = tid >> 3;
  const int col = blockIdx.x * kSCols + cl;
  const bool live = col < dv;
  const long y_stride = (long)heads * dv;
  if (sl < 0 || sl >= num_slots) {
    if (live && kl == 0)
      for (int t = 0; t < rows; ++t) y[(long)(r0 + t) * y_stride + (long)h * dv + col] = 0.f;
    return;
  }
  if (rows <= 0) return;
  const int g = h / (heads / groups);
  const int c = live ? col : dv - 1;      // dead lanes shadow the last column, store nothing
  float* S = state + (((long)sl * heads + h) * n) * dv;
  float st_[R];
  const bool fresh = pos0[s] <= 0;
#pragma unroll
  for (int r = 0; r < R; ++r) st_[r] = (!fresh && kl + kSL * r < n) ? S[(long)(kl + kSL * r) * dv + c] : 0.f;
  const long xoff = (long)h * dv + (long)blockIdx.x * kSCols;
  const long boff = (long)heads * dv + (long)g * n;
  const long coff = boff + (long)groups * n;
  const float rate = expf(a_log[h]), bias = dt_bias[h], skip = d_skip[h];

  float ld_[P::NLD], lv_[P::NV], lstep_ = 0.f, ldec_ = 0.f;
  auto fetch = [&](int t0, int cnt) {
#pragma unroll
    for (int u = 0; u < P::NLD; ++u) {
      const int e = tid + 256 * u;                  // (row tt, array a, entry i) of the chunk
      const int tt = e / (2 * P::NP), rem = e % (2 * P::NP);
      const int a = rem / P::NP, i = rem % P::NP;
      float v = 0.f;
      if (tt < cnt && i < n) v = ld(xbc, (long)(r0 + t0 + tt) * x_stride + (a == 0 ? boff : coff) + i);
      ld_[u] = v;
    }
#pragma unroll
    for (int u = 0; u < P::NV; ++u) {
      const int e = tid + 256 * u;
      const int tt = e / kSCols, cc = e % kSCols;
      lv_[u] = (tt < cnt && blockIdx.x * kSCols + cc < dv) ? ld(xbc, (long)(r0 + t0 + tt) * x_stride + xoff + cc)
                                                           : 0.f;
    }
    if (tid < cnt) {
      lstep_ = softplusf_(ld(dt, (long)(r0 + t0 + tid) * dt_stride + h) + bias);
      ldec_ = expf(-rate * lstep_);
    }
  };
  auto park = [&](float* buf) {
#pragma unroll
    for (int u = 0; u < P::NLD; ++u) {
      const int e = tid + 256 * u;
      const int tt = e / (2 * P::NP), rem = e % (2 * P::NP);
      if (tt < P::TT) buf[tt * P::ROWF + rem] = ld_[u];
    }
#pragma unroll
    for (int u = 0; u < P::NV; ++u) {
      const int e = tid + 256 * u;
      if (e < P::TT * kSCols) buf[(e / kSCols) * P::ROWF + 2 * P::NP + e % kSCols] = lv_[u];
    }
    if (tid < P::TT) {
      buf[tid * P::ROWF + 2 * P::NP + kSCols] = lstep_;
      buf[tid * P::ROWF + 2 * P::NP + kSCols + 1] = ldec_;
    }
  };

  fetch(0, min(P::TT, rows));
  park(stage[0]);
  __syncthreads();
  int cur = 0;
  for (int t0 = 0; t0 < rows; t0 += P::TT) {
    const int cnt = min(P::TT, rows - t0);
    const bool more = t0 + P::TT < rows;
    if (more) fetch(t0 + P::TT, min(P::TT, rows - t0 - P::TT));
    const float* buf = stage[cur];
    for (int t = 0; t < cnt; ++t) {
      const float* rw = buf + t * P::ROWF;
      const float xv = rw[2 * P::NP + cl];
      const float dec = rw[2 * P::NP + kSCols + 1];
      const float sx = rw[2 * P::NP + kSCols] * xv;
      float out = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        st_[r] = dec * st_[r] + rw[kl + kSL * r] * sx;
        out += st_[r] * rw[P::NP + kl + kSL * r];
      }
      out = ssd_sum8(out);
      if (live && kl == 0) y[(long)(r0 + t0 + t) * y_stride + (long)h * dv + col] = out + skip * xv;
    }
    if (more) park(stage[cur ^ 1]);
    __syncthreads();
    cur ^= 1;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (kl + kSL * r < n) S[(long)(kl + kSL * r) * dv + col] = st_[r];
  }
}

// one wave per (row, group): v = y * silu(z); out = v / rms(v) * w
template <typename TZ, typename TO>
__global__ void gate_group_norm_kernel(TO* __restrict__ out, const float* __restrict__ y, const TZ* __restrict__ z,
                                       long z_stride, const float* __restrict__ w, long pairs, int groups, int gs,
                                       float eps) {
  const long pair = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const long row = pair / groups;
  const int g = (int)(pair % groups);
  const long width = (long)groups * gs;
  const float* yp = y + row * width + (long)g * gs;
  const TZ* zp = z + row * z_stride + (long)g * gs;
  float ss = 0.f;
  for (int c = lane; c < gs; c += 64) {
    const float zv = ld(zp, c);
    const float v = yp[c] * (zv * sigmoidf_(zv));
    ss += v * v;
  }
  ss = ft::wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)gs + eps);
  for (int c = lane; c < gs; c += 64) {
    const float zv = ld(zp, c);
    st(out, row * width + (long)g * gs + c, yp[c] * (zv * sigmoidf_(zv)) * r * w[(long)g * gs + c]);
  }
}

}  // namespace mx

using namespace mx;

extern "C" int mx_ssd_max_state() { return kSL * 32; }

template <typename T, int R>
static void launch_ssd(dim3 grid, hipStream_t s, float* y, const void* xbc, long x_stride, const void* dt,
                       long dt_stride, const float* a_log, const float* dt_bias, const float* d_skip, float* state,
                       const int* start, const int* pos0, const int* slot, int heads, int groups, int n, int dv,
                       int num_slots) {
  hipLaunchKernelGGL((ssd_scan_kernel<T, R>), grid, dim3(256), 0, s, y, (const T*)xbc, x_stride, (const T*)dt,
                     dt_stride, a_log, dt_bias, d_skip, state, start, pos0, slot, heads, groups, n, dv, num_slots);
}

extern "C" int mx_ssd_scan(float* y, const void* xbc, int bf16, long x_stride, const void* dt, long dt_stride,
                           const float* a_log, const float* dt_bias, const float* d_skip, float* state,
                           const int* start, const int* pos0, const int* slot, int num_segs, int heads, int groups,
                           int n, int dv, int num_slots, hipStream_t s) {
  if (num_segs <= 0) return 0;
  if (n < 1 || n > mx_ssd_max_state() || dv < 1 || groups < 1 || heads % groups) return -1;
  const dim3 grid((dv + kSCols - 1) / kSCols, heads, num_segs);
  if (grid.z > 65535 || grid.y > 65535) return -2;
  const int need = (n + kSL - 1) / kSL;
#define MX_SSD(R)                                                                                         \
  MX_DISPATCH_T(bf16, launch_ssd<T, R>(grid, s, y, xbc, x_stride, dt, dt_stride, a_log, dt_bias, d_skip, state, \
                                       start, pos0, slot, heads, groups, n, dv, num_slots))
  if (need <= 2) MX_SSD(2);
  else if (need <= 4) MX_SSD(4);
  else if (need <= 8) MX_SSD(8);
  else if (need <= 16) MX_SSD(16);
  else MX_SSD(32);
#undef MX_SSD
  return (int)hipGetLastError();
}

extern "C" int mx_gate_group_norm(void* out, int out_bf16, const float* y, const void* z, int z_bf16, long z_stride,
                                  const float* w, long rows, int groups, int gs, float eps, hipStream_t s) {
  const long pairs = rows * groups;
  if (pairs <= 0) return 0;
  const dim3 grid((unsigned)((pairs + 3) / 4)), block(256);
  if (z_bf16 && out_bf16)
    hipLaunchKernelGGL((gate_group_norm_kernel<bf16_t, bf16_t>), grid, block, 0, s, (bf16_t*)out, y,
                       (const bf16_t*)z, z_stride, w, pairs, groups, gs, eps);
  else if (!z_bf16 && !out_bf16)
    hipLaunchKernelGGL((gate_group_norm_kernel<float, float>), grid, block, 0, s, (float*)out, y, (const float*)z,
                       z_stride, w, pairs, groups, gs, eps);
  else
    return -1;
  return (int)hipGetLastError();
}
