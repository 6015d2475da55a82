// Selective state-space scan with one scalar decay per head and row over fp32 state
// slots, and the gated grouped RMS norm that follows it.
//
// Rows come in segments as in delta_rule.hip (start / pos0 / slot; a segment at
// position 0 starts from zeros; slot < 0 is padding).  Rows of xbc are
// [x (heads*dv) | B (groups*n) | C (groups*n)].  Per head h (group h / (heads/groups)):
//   step = softplus(dt + dt_bias[h]);  decay = exp(-exp(a_log[h]) * step)
//   S <- decay S + step B x^T   (S is n x dv);   y = S^T C + d_skip[h] x
// Columns of S are independent, so a workgroup owns 16 columns of one head of one
// sequence: 16 lanes share a column, lane kl holding the R consecutive state rows
// kl R .. kl R + R - 1 in registers (n <= 16 R), the output dot product reduced over
// those 16 lanes; a segment's rows are walked in order with the per-row inputs staged
// through LDS in double-buffered chunks.  A lane's R entries of B and of C lie together
// in LDS (16-byte reads; the 16 lanes' runs are padded apart so they fall into different
// banks), and a full chunk's walk is unrolled so the reads of the next rows are issued
// under the current row's arithmetic.
#include "mx_common.h"

namespace mx {

constexpr int kSL = 16;        // lanes that share one state column (one DPP row)
constexpr int kSCols = 16;     // state columns per workgroup (256 threads)

// sum over the 16 lanes of a DPP row: every lane gets the total
__device__ __forceinline__ float ssd_sum16(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // lanes ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // lanes ^ 2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // 7 - lane (halves)
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));  // 15 - lane
  return v;
}

template <int R>
struct SsdTile {
  static constexpr int TT = R <= 8 ? 16 : 8;                  // rows per chunk
  static constexpr int NP = kSL * R;                          // padded state size
  static constexpr int SR = R + (R >= 8 ? 4 : 0);             // floats between two lanes' runs of B (or C)
  static constexpr int BP = kSL * SR;                         // floats of a staged B (or C)
  static constexpr int ROWF = 2 * BP + kSCols + 4;            // floats per staged row: B | C | x | step, decay, -, -
  static constexpr int NLD = (TT * 2 * NP + 255) / 256;       // B/C loads per thread and chunk
  static constexpr int NV = (TT * kSCols + 255) / 256;        // x loads per thread and chunk
};

// R consecutive floats from LDS (16-byte aligned when R >= 4)
template <int R>
__device__ __forceinline__ void lds_run(const float* p, float* v) {
  if constexpr (R >= 4) {
#pragma unroll
    for (int i = 0; i < R / 4; ++i) {
      const float4 u = reinterpret_cast<const float4*>(p)[i];
      v[4 * i] = u.x; v[4 * i + 1] = u.y; v[4 * i + 2] = u.z; v[4 * i + 3] = u.w;
    }
  } else {
    const float2 u = *reinterpret_cast<const float2*>(p);
    v[0] = u.x; v[1] = u.y;
  }
}

template <typename T, int R>
__global__ void __launch_bounds__(256)
ssd_scan_kernel(float* __restrict__ y, const T* __restrict__ xbc, long x_stride, const T* __restrict__ dt,
                long dt_stride, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                const float* __restrict__ d_skip, float* __restrict__ state, const int* __restrict__ start,
                const int* __restrict__ pos0, const int* __restrict__ slot, int heads, int groups, int n,
                int dv, int num_slots) {
  using P = SsdTile<R>;
  __shared__ __attribute__((aligned(16))) float stage[2][P::TT * P::ROWF];
  __shared__ float out_s[2][P::TT * kSCols];     // a chunk's outputs, written out after the walk
  const int s = blockIdx.z, h = blockIdx.y;
  const int sl = slot[s];
  const int r0 = start[s], rows = start[s + 1] - r0;
  const int tid = threadIdx.x;
  const int kl = tid & (kSL - 1);
  const int cl = tid / kSL;
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
  for (int r = 0; r < R; ++r) st_[r] = (!fresh && kl * R + r < n) ? S[(long)(kl * R + r) * dv + c] : 0.f;
  const long xoff = (long)h * dv + (long)blockIdx.x * kSCols;
  const long boff = (long)heads * dv + (long)g * n;
  const long coff = boff + (long)groups * n;
  const float rate = expf(a_log[h]), bias = dt_bias[h], skip = d_skip[h];

  // the next chunk's inputs are loaded raw (no use of the values, so no wait for them
  // before the walk) and converted when they are parked in LDS after the walk
  T ld_[P::NLD], lv_[P::NV], ldt_ = T(0);
  auto fetch = [&](int t0, int cnt) {
#pragma unroll
    for (int u = 0; u < P::NLD; ++u) {
      const int e = tid + 256 * u;                  // (row tt, array a, entry i) of the chunk
      const int tt = e / (2 * P::NP), rem = e % (2 * P::NP);
      const int a = rem / P::NP, i = rem % P::NP;
      T v = T(0);
      if (tt < cnt && i < n) v = xbc[(long)(r0 + t0 + tt) * x_stride + (a == 0 ? boff : coff) + i];
      ld_[u] = v;
    }
#pragma unroll
    for (int u = 0; u < P::NV; ++u) {
      const int e = tid + 256 * u;
      const int tt = e / kSCols, cc = e % kSCols;
      lv_[u] = (tt < cnt && blockIdx.x * kSCols + cc < dv) ? xbc[(long)(r0 + t0 + tt) * x_stride + xoff + cc] : T(0);
    }
    if (tid < cnt) ldt_ = dt[(long)(r0 + t0 + tid) * dt_stride + h];
  };
  auto park = [&](float* buf) {
#pragma unroll
    for (int u = 0; u < P::NLD; ++u) {
      const int e = tid + 256 * u;
      const int tt = e / (2 * P::NP), rem = e % (2 * P::NP);
      const int a = rem / P::NP, i = rem % P::NP;
      if (tt < P::TT) buf[tt * P::ROWF + a * P::BP + (i / R) * P::SR + i % R] = ld(&ld_[u], 0);
    }
#pragma unroll
    for (int u = 0; u < P::NV; ++u) {
      const int e = tid + 256 * u;
      if (e < P::TT * kSCols) buf[(e / kSCols) * P::ROWF + 2 * P::BP + e % kSCols] = ld(&lv_[u], 0);
    }
    if (tid < P::TT) {
      const float step = softplusf_(ld(&ldt_, 0) + bias);
      buf[tid * P::ROWF + 2 * P::BP + kSCols] = step;
      buf[tid * P::ROWF + 2 * P::BP + kSCols + 1] = expf(-rate * step);
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
    auto walk = [&](int t) {
      const float* rw = buf + t * P::ROWF;
      float bb[R], cc[R];
      lds_run<R>(rw + kl * P::SR, bb);
      lds_run<R>(rw + P::BP + kl * P::SR, cc);
      const float xv = rw[2 * P::BP + cl];
      const float dec = rw[2 * P::BP + kSCols + 1];
      const float sx = rw[2 * P::BP + kSCols] * xv;
      float part[R >= 4 ? 4 : R];                   // independent partial sums: short dependency chains
#pragma unroll
      for (int r = 0; r < R; ++r) {
        st_[r] = dec * st_[r] + bb[r] * sx;
        if (r < 4) part[r] = st_[r] * cc[r];
        else part[r & 3] += st_[r] * cc[r];
      }
      float out = part[0];
#pragma unroll
      for (int r = 1; r < (R >= 4 ? 4 : R); ++r) out += part[r];
      out = ssd_sum16(out);
      if (kl == 0) out_s[cur][t * kSCols + cl] = out + skip * xv;
    };
    if (cnt == P::TT) {
#pragma unroll
      for (int t = 0; t < P::TT; ++t) walk(t);
    } else {
      for (int t = 0; t < cnt; ++t) walk(t);
    }
    if (more) park(stage[cur ^ 1]);
    __syncthreads();
    // the chunk's outputs: one coalesced store per thread (rows of 16 columns)
    if (tid < cnt * kSCols) {
      const int tt = tid / kSCols, cc = tid % kSCols;
      if (blockIdx.x * kSCols + cc < dv)
        y[(long)(r0 + t0 + tt) * y_stride + (long)h * dv + blockIdx.x * kSCols + cc] = out_s[cur][tid];
    }
    cur ^= 1;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (kl * R + r < n) S[(long)(kl * R + r) * dv + col] = st_[r];
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

extern "C" int mx_ssd_max_state() { return kSL * 16; }

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
  else MX_SSD(16);
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
