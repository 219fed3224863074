// seq_linear.hip -- dihip_linear: y = epilogue(x . W^T + bias) for row-major [N, K] weights as checkpoints store them,
// grouped (block-diagonal / per-head) forms included.  Three kernels:
//   linear_tile_kernel   every product and sum in f32, k ascending (DIHIP_MATH_F32; also any operand type / odd shape)
//   linear_mfma_kernel   bf16 operands on the 16x16x32 matrix-core tiles, 128 x 128 x 32 block tiles, f32 accumulation
//   linear_skinny_kernel up to 4 rows at a time against a streamed weight (decode): one wave per 4 weight rows
// An output element is computed by one thread (or one MFMA column) over k in a fixed order: it does not depend on T.
#include "seq_common.h"

namespace dihip {
namespace {

struct LinArgs {
  const void* x; long ldx, xg; int xgroups;
  const void* w; const void* bias;
  void* y; long ldy, yg;
  const float* mul; long ldm;
  int T, N, K, act, act_lo, act_hi, ydt, round_ops;
  const int32_t* seg; const int32_t* row_map;   // segmented form: group g owns the output rows seg[g] .. seg[g + 1], row r reads x row row_map[r]
};

// the rows of group g: [lo, hi)
__device__ __forceinline__ void lin_rows(const LinArgs& a, int g, int& lo, int& hi) {
  lo = 0; hi = a.T;
  if (a.seg) { lo = a.seg[g]; hi = a.seg[g + 1]; }
}
__device__ __forceinline__ size_t lin_xrow(const LinArgs& a, int r) { return (size_t)(a.row_map ? a.row_map[r] : r); }

__device__ __forceinline__ void lin_epilogue(const LinArgs& a, int g, int t, int n, float v, int wdt) {
  if (a.bias) v += ld_any(a.bias, (size_t)g * a.N + n, wdt);
  const int col = g * a.N + n;
  if (col >= a.act_lo && col < a.act_hi) v = apply_act(v, a.act);
  const size_t o = (size_t)t * a.ldy + (size_t)g * a.yg + n;
  if (a.mul) v *= a.mul[(size_t)t * a.ldm + (size_t)g * a.yg + n];
  st_any(a.y, o, a.ydt, v);
}

// ------------------------------------------------------------------------------------------ exact f32 tile kernel
template <int XT, int WT>
__global__ __launch_bounds__(256) void linear_tile_kernel(LinArgs a) {
  __shared__ float xs[16][68];
  __shared__ float ws[16][68];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int g = blockIdx.z, n0 = blockIdx.x * 64;
  int t_lo, t_hi;
  lin_rows(a, g, t_lo, t_hi);
  const int m0 = t_lo + blockIdx.y * 64;
  if (m0 >= t_hi) return;
  const size_t xoff = (size_t)(g % a.xgroups) * a.xg;
  const size_t wbase = (size_t)g * a.N * a.K;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < a.K; k0 += 16) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int idx = tid + 256 * j, r = idx >> 4, kk = idx & 15;
      float xv = 0.f, wv = 0.f;
      if (k0 + kk < a.K) {
        if (m0 + r < t_hi) xv = load_ft<XT>(a.x, lin_xrow(a, m0 + r) * a.ldx + xoff + k0 + kk);
        if (n0 + r < a.N) wv = load_ft<WT>(a.w, wbase + (size_t)(n0 + r) * a.K + k0 + kk);
      }
      if (a.round_ops) { xv = ft_round<DIHIP_BF16>(xv); wv = ft_round<DIHIP_BF16>(wv); }
      xs[kk][r] = xv;
      ws[kk][r] = wv;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      const f32x4_t av = *reinterpret_cast<const f32x4_t*>(&xs[kk][ty * 4]);
      const f32x4_t bv = *reinterpret_cast<const f32x4_t*>(&ws[kk][tx * 4]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = m0 + ty * 4 + i;
    if (t >= t_hi) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < a.N) lin_epilogue(a, g, t, n, acc[i][j], WT);
    }
  }
}

// ------------------------------------------------------------------------------------------ bf16 matrix-core kernel
__device__ __forceinline__ f32x4_t mfma_bf16(const u32x4_t& a, const u32x4_t& b, const f32x4_t& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// 8 consecutive k of one row as packed bf16; VEC: the 8 are in range and 16-byte aligned (host-checked), else guarded
template <int XT, bool VEC>
__device__ __forceinline__ u32x4_t load8_bf16(const void* p, size_t i, int kleft, bool row_ok) {
  u32x4_t r = {0u, 0u, 0u, 0u};
  if (!row_ok || kleft <= 0) return r;
  if constexpr (VEC) {
    if constexpr (XT == DIHIP_F32) {
      const f32x4_t lo = *reinterpret_cast<const f32x4_t*>((const float*)p + i);
      const f32x4_t hi = *reinterpret_cast<const f32x4_t*>((const float*)p + i + 4);
      r[0] = pack_bf16x2(lo[0], lo[1]); r[1] = pack_bf16x2(lo[2], lo[3]);
      r[2] = pack_bf16x2(hi[0], hi[1]); r[3] = pack_bf16x2(hi[2], hi[3]);
    } else {
      r = *reinterpret_cast<const u32x4_t*>((const uint16_t*)p + i);
    }
  } else {
    uint32_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = j < kleft ? f32_to_bf16_bits(load_ft<XT>(p, i + j)) : 0u;
    r[0] = e[0] | (e[1] << 16); r[1] = e[2] | (e[3] << 16); r[2] = e[4] | (e[5] << 16); r[3] = e[6] | (e[7] << 16);
  }
  return r;
}

template <int XT, bool VEC>
__global__ __launch_bounds__(256) void linear_mfma_kernel(LinArgs a) {
  constexpr int BK = 32, UPR = BK / 8, UN = 128 * UPR / 256;   // k per step (64 measured slower: fewer workgroups per CU), 16-byte units per tile row, units per thread
  constexpr int LD = BK + 8;  // bf16 elements per LDS row: 8 of padding (80 bytes: 16-byte aligned fragments)
  __shared__ __attribute__((aligned(16))) uint16_t As[128 * LD];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[128 * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int g = blockIdx.z, n0 = blockIdx.x * 128;
  int t_lo, t_hi;
  lin_rows(a, g, t_lo, t_hi);
  const int m0 = t_lo + blockIdx.y * 128;
  if (m0 >= t_hi) return;
  const size_t xoff = (size_t)(g % a.xgroups) * a.xg;
  const size_t wbase = (size_t)g * a.N * a.K;
  const f32x4_t z4 = {0.f, 0.f, 0.f, 0.f};
  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = z4;
  u32x4_t ra[UN], rb[UN];
  size_t xrow[UN];   // the x row of each of the thread's units: fixed for the whole walk
#pragma unroll
  for (int j = 0; j < UN; ++j) {
    const int r = (tid + 256 * j) / UPR;
    xrow[j] = m0 + r < t_hi ? lin_xrow(a, m0 + r) : 0;
  }
  auto fetch = [&](int k0) {
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      const int u = tid + 256 * j, r = u / UPR, k = k0 + (u % UPR) * 8;
      ra[j] = load8_bf16<XT, VEC>(a.x, xrow[j] * a.ldx + xoff + k, a.K - k, m0 + r < t_hi);
      rb[j] = load8_bf16<DIHIP_BF16, VEC>(a.w, wbase + (size_t)(n0 + r) * a.K + k, a.K - k, n0 + r < a.N);
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < a.K; k0 += BK) {
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      const int u = tid + 256 * j, r = u / UPR, kq = (u % UPR) * 8;
      *reinterpret_cast<u32x4_t*>(&As[r * LD + kq]) = ra[j];
      *reinterpret_cast<u32x4_t*>(&Bs[r * LD + kq]) = rb[j];
    }
    __syncthreads();
    if (k0 + BK < a.K) fetch(k0 + BK);
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      u32x4_t af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        af[i] = *reinterpret_cast<const u32x4_t*>(&As[(wm * 64 + i * 16 + (lane & 15)) * LD + ks * 32 + (lane >> 4) * 8]);
        bf[i] = *reinterpret_cast<const u32x4_t*>(&Bs[(wn * 64 + i * 16 + (lane & 15)) * LD + ks * 32 + (lane >> 4) * 8]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mfma_bf16(af[i], bf[j], acc[i][j]);
    }
    __syncthreads();
  }
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");  // the matrix pipe's write-back before the results are read
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + wn * 64 + j * 16 + (lane & 15);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = m0 + wm * 64 + i * 16 + (lane >> 4) * 4 + r;
        if (t < t_hi && n < a.N) lin_epilogue(a, g, t, n, acc[i][j][r], DIHIP_BF16);
      }
    }
}

// ------------------------------------------------------------------------------------------ weight-streaming kernel
__device__ __forceinline__ float dot8_bf16(const u32x4_t& w, const u32x4_t& x, float acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    acc = __builtin_fmaf(__uint_as_float(w[i] << 16), __uint_as_float(x[i] << 16), acc);
    acc = __builtin_fmaf(__uint_as_float(w[i] & 0xffff0000u), __uint_as_float(x[i] & 0xffff0000u), acc);
  }
  return acc;
}

// rows t0 .. t0 + tc (tc <= 4) of x staged in LDS -- as bf16, or as they are (EXACT: f32 products of the unrounded row) --;
// wave w of block b owns weight rows (b * 4 + w) * 2 .. + 2 and keeps two 1 KiB slices of each in flight.
// K % 8 == 0 and 16-byte aligned weight rows (host-checked).
template <int XT, bool EXACT>
__global__ __launch_bounds__(256) void linear_skinny_kernel(LinArgs a, int t0, int tc) {
  if (a.seg) {   // rows t0 .. of the group's own segment (block-uniform)
    const int lo = a.seg[blockIdx.y] + t0, left = a.seg[blockIdx.y + 1] - lo;
    if (left <= 0) return;
    t0 = lo;
    tc = min(tc, left);
  }
  extern __shared__ __attribute__((aligned(16))) unsigned char xraw[];
  uint16_t* xsm = reinterpret_cast<uint16_t*>(xraw);
  float* xsf = reinterpret_cast<float*>(xraw);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = blockIdx.y;
  const size_t xoff = (size_t)(g % a.xgroups) * a.xg;
  const int nb = (blockIdx.x * 4 + wave) * 2;
  const bool mine = nb < a.N;
  const uint16_t* wp = (const uint16_t*)a.w + (size_t)g * a.N * a.K;
  const uint16_t* w0 = wp + (size_t)min(nb, a.N - 1) * a.K;
  const uint16_t* w1 = wp + (size_t)min(nb + 1, a.N - 1) * a.K;
  const u32x4_t z = {0u, 0u, 0u, 0u};
  u32x4_t cur[2][2], nxt[2][2];
  auto wload = [&](u32x4_t (&d)[2][2], int k) {   // two 1 KiB slices of both rows, zeros beyond K
    const bool one = k < a.K, two = k + 512 < a.K;
    d[0][0] = one ? *reinterpret_cast<const u32x4_t*>(w0 + k) : z;
    d[1][0] = one ? *reinterpret_cast<const u32x4_t*>(w1 + k) : z;
    d[0][1] = two ? *reinterpret_cast<const u32x4_t*>(w0 + k + 512) : z;
    d[1][1] = two ? *reinterpret_cast<const u32x4_t*>(w1 + k + 512) : z;
  };
  wload(cur, lane * 8);     // in flight while the rows are staged
  // staging in units of 8 elements (K % 8 == 0, 16-byte aligned rows: host-checked), several units of a thread in flight
  const int upr = a.K >> 3, units = tc * upr;
#pragma unroll 4
  for (int u = tid; u < units; u += 256) {
    const int t = u / upr, k = (u - t * upr) * 8;
    const size_t src = lin_xrow(a, t0 + t) * a.ldx + xoff + k;
    float v[8];
    if constexpr (XT == DIHIP_F32) {
      const f32x4_t lo = *reinterpret_cast<const f32x4_t*>((const float*)a.x + src);
      const f32x4_t hi = *reinterpret_cast<const f32x4_t*>((const float*)a.x + src + 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) { v[j] = lo[j]; v[4 + j] = hi[j]; }
    } else {
      const u32x4_t r = *reinterpret_cast<const u32x4_t*>((const uint16_t*)a.x + src);
#pragma unroll
      for (int j = 0; j < 4; ++j) { v[2 * j] = __uint_as_float(r[j] << 16); v[2 * j + 1] = __uint_as_float(r[j] & 0xffff0000u); }
    }
    if constexpr (EXACT) {
      *reinterpret_cast<f32x4_t*>(xsf + (size_t)t * a.K + k) = f32x4_t{v[0], v[1], v[2], v[3]};
      *reinterpret_cast<f32x4_t*>(xsf + (size_t)t * a.K + k + 4) = f32x4_t{v[4], v[5], v[6], v[7]};
    } else {
      *reinterpret_cast<u32x4_t*>(xsm + (size_t)t * a.K + k) =
          u32x4_t{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])};
    }
  }
  __syncthreads();
  if (!mine) return;
  float acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[i][t] = 0.f;
  for (int k = lane * 8; k < a.K; k += 1024) {
    wload(nxt, k + 1024);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kk = k + h * 512;
      if (kk >= a.K) break;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        if (t < tc) {
          if constexpr (EXACT) {
            const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(xsf + (size_t)t * a.K + kk);
            const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(xsf + (size_t)t * a.K + kk + 4);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
              float v = acc[i][t];
              v = __builtin_fmaf(__uint_as_float(cur[i][h][0] << 16), lo[0], v);
              v = __builtin_fmaf(__uint_as_float(cur[i][h][0] & 0xffff0000u), lo[1], v);
              v = __builtin_fmaf(__uint_as_float(cur[i][h][1] << 16), lo[2], v);
              v = __builtin_fmaf(__uint_as_float(cur[i][h][1] & 0xffff0000u), lo[3], v);
              v = __builtin_fmaf(__uint_as_float(cur[i][h][2] << 16), hi[0], v);
              v = __builtin_fmaf(__uint_as_float(cur[i][h][2] & 0xffff0000u), hi[1], v);
              v = __builtin_fmaf(__uint_as_float(cur[i][h][3] << 16), hi[2], v);
              v = __builtin_fmaf(__uint_as_float(cur[i][h][3] & 0xffff0000u), hi[3], v);
              acc[i][t] = v;
            }
          } else {
            const u32x4_t xv = *reinterpret_cast<const u32x4_t*>(xsm + (size_t)t * a.K + kk);
#pragma unroll
            for (int i = 0; i < 2; ++i) acc[i][t] = dot8_bf16(cur[i][h], xv, acc[i][t]);
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int h = 0; h < 2; ++h) cur[i][h] = nxt[i][h];
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float v = wave_sum(acc[i][t]);
      if (lane == 0 && t < tc && nb + i < a.N) lin_epilogue(a, g, t0 + t, nb + i, v, DIHIP_BF16);
    }
}

// Few output columns against many rows (a router's logits): one workgroup per row, the row staged in LDS as f32, a wave per
// column: f32 products of the unrounded row, each lane over its k in ascending order, then the fixed tree over the lanes.
// K % 8 == 0 and 16-byte aligned weight rows (host-checked).
template <int XT>
__global__ __launch_bounds__(256) void linear_fewcols_kernel(LinArgs a) {
  extern __shared__ __attribute__((aligned(16))) float xrow[];
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int k = tid; k < a.K; k += 256) xrow[k] = load_ft<XT>(a.x, (size_t)t * a.ldx + k);
  __syncthreads();
  for (int n = wave; n < a.N; n += 4) {
    const uint16_t* wr = (const uint16_t*)a.w + (size_t)n * a.K;
    float acc = 0.f;
    for (int k = lane * 8; k < a.K; k += 512) {
      const u32x4_t wv = *reinterpret_cast<const u32x4_t*>(wr + k);
      const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(xrow + k), hi = *reinterpret_cast<const f32x4_t*>(xrow + k + 4);
      acc = __builtin_fmaf(__uint_as_float(wv[0] << 16), lo[0], acc);
      acc = __builtin_fmaf(__uint_as_float(wv[0] & 0xffff0000u), lo[1], acc);
      acc = __builtin_fmaf(__uint_as_float(wv[1] << 16), lo[2], acc);
      acc = __builtin_fmaf(__uint_as_float(wv[1] & 0xffff0000u), lo[3], acc);
      acc = __builtin_fmaf(__uint_as_float(wv[2] << 16), hi[0], acc);
      acc = __builtin_fmaf(__uint_as_float(wv[2] & 0xffff0000u), hi[1], acc);
      acc = __builtin_fmaf(__uint_as_float(wv[3] << 16), hi[2], acc);
      acc = __builtin_fmaf(__uint_as_float(wv[3] & 0xffff0000u), hi[3], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) lin_epilogue(a, 0, t, n, acc, DIHIP_BF16);
  }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace
}  // namespace dihip

using namespace dihip;

static int linear_impl(void* stream, const void* x, int x_dtype, long ldx, long x_gstride, int x_groups, const void* w,
                       int w_dtype, const void* bias, void* y, int y_dtype, long ldy, long y_gstride, const float* mul,
                       long ldm, int T, int N, int K, int groups, int act, int act_lo, int act_hi, int math,
                       const int32_t* seg, const int32_t* row_map, int seg_max_rows) {
  DIHIP_REQUIRE(T >= 0 && N > 0 && K > 0 && groups > 0 && x_groups > 0, DIHIP_PARAM_ERROR, "linear: bad shape T %d N %d K %d groups %d", T, N, K, groups);
  DIHIP_REQUIRE(seq_dtype_ok(x_dtype) && seq_dtype_ok(w_dtype) && seq_dtype_ok(y_dtype), DIHIP_PARAM_ERROR, "linear: f32 / bf16 only");
  DIHIP_REQUIRE(x && w && y, DIHIP_PARAM_ERROR, "linear: null pointer");
  DIHIP_REQUIRE(ldx >= K && ldy >= N && (!mul || ldm >= N), DIHIP_PARAM_ERROR, "linear: a row stride below the row length");
  DIHIP_REQUIRE(math == DIHIP_MATH_F32 || math == DIHIP_MATH_BF16 || math == DIHIP_MATH_F32_STREAM, DIHIP_PARAM_ERROR,
                "linear: unknown math mode %d", math);
  DIHIP_REQUIRE(groups <= 65535, DIHIP_PARAM_ERROR, "linear: more than 65535 groups");
  if (T == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  LinArgs a{x, ldx, x_gstride, x_groups, w, bias, y, ldy, y_gstride, mul, ldm, T, N, K, act, act_lo, act_hi, y_dtype, 0, seg, row_map};
  const int Tg = seg ? (seg_max_rows < T ? seg_max_rows : T) : T;   // the most rows one group can have
  const size_t xe = x_dtype == DIHIP_F32 ? 4 : 2;
  const bool vec = w_dtype == DIHIP_BF16 && K % 8 == 0 && aligned16(w) && aligned16(x) && (ldx * xe) % 16 == 0 &&
                   (x_gstride * xe) % 16 == 0;
  static const bool no_skinny = env_off("DIHIP_LINEAR_SKINNY");
  if (math == DIHIP_MATH_F32_STREAM) {
    // f32 products of unrounded rows; few rows stream the weight once (a row's sum then runs in the lanes' order, not k ascending)
    const int tmax = K <= 4096 ? 4 : (K <= 8192 ? 2 : 1);
    if (Tg <= 4 * tmax && vec && !no_skinny && K <= 16384) {
      for (int t0 = 0; t0 < Tg; t0 += tmax) {
        const int tc = Tg - t0 < tmax ? Tg - t0 : tmax;
        const dim3 grid((N + 7) / 8, groups);
        if (x_dtype == DIHIP_F32) hipLaunchKernelGGL((linear_skinny_kernel<DIHIP_F32, true>), grid, dim3(256), (size_t)tc * K * 4, s, a, t0, tc);
        else hipLaunchKernelGGL((linear_skinny_kernel<DIHIP_BF16, true>), grid, dim3(256), (size_t)tc * K * 4, s, a, t0, tc);
      }
      return launch_status();
    }
    if (N <= 64 && groups == 1 && !seg && vec && K <= 16384) {   // many rows, few columns: the tile kernel would idle most of its 64 x 64 tile
      if (x_dtype == DIHIP_F32) hipLaunchKernelGGL((linear_fewcols_kernel<DIHIP_F32>), dim3(T), dim3(256), (size_t)K * 4, s, a);
      else hipLaunchKernelGGL((linear_fewcols_kernel<DIHIP_BF16>), dim3(T), dim3(256), (size_t)K * 4, s, a);
      return launch_status();
    }
    math = DIHIP_MATH_F32;
  }
  if (math == DIHIP_MATH_BF16 && w_dtype == DIHIP_BF16) {
    const int tmax = K <= 8192 ? 4 : (K <= 16384 ? 2 : 1);  // rows whose bf16 copy fits 64 KB of LDS
    if (Tg <= 4 * tmax && vec && !no_skinny && K <= 32768) {
      for (int t0 = 0; t0 < Tg; t0 += tmax) {
        const int tc = Tg - t0 < tmax ? Tg - t0 : tmax;
        const dim3 grid((N + 7) / 8, groups);
        if (x_dtype == DIHIP_F32) hipLaunchKernelGGL((linear_skinny_kernel<DIHIP_F32, false>), grid, dim3(256), (size_t)tc * K * 2, s, a, t0, tc);
        else hipLaunchKernelGGL((linear_skinny_kernel<DIHIP_BF16, false>), grid, dim3(256), (size_t)tc * K * 2, s, a, t0, tc);
      }
      return launch_status();
    }
    const dim3 grid((N + 127) / 128, (Tg + 127) / 128, groups);
    DIHIP_REQUIRE(grid.y <= 65535, DIHIP_PARAM_ERROR, "linear: too many rows for one launch");
    if (x_dtype == DIHIP_F32) {
      if (vec) hipLaunchKernelGGL((linear_mfma_kernel<DIHIP_F32, true>), grid, dim3(256), 0, s, a);
      else hipLaunchKernelGGL((linear_mfma_kernel<DIHIP_F32, false>), grid, dim3(256), 0, s, a);
    } else {
      if (vec) hipLaunchKernelGGL((linear_mfma_kernel<DIHIP_BF16, true>), grid, dim3(256), 0, s, a);
      else hipLaunchKernelGGL((linear_mfma_kernel<DIHIP_BF16, false>), grid, dim3(256), 0, s, a);
    }
    return launch_status();
  }
  a.round_ops = math == DIHIP_MATH_BF16;
  const dim3 grid((N + 63) / 64, (Tg + 63) / 64, groups);
  DIHIP_REQUIRE(grid.y <= 65535, DIHIP_PARAM_ERROR, "linear: too many rows for one launch");
  if (x_dtype == DIHIP_F32 && w_dtype == DIHIP_F32) hipLaunchKernelGGL((linear_tile_kernel<DIHIP_F32, DIHIP_F32>), grid, dim3(256), 0, s, a);
  else if (x_dtype == DIHIP_F32) hipLaunchKernelGGL((linear_tile_kernel<DIHIP_F32, DIHIP_BF16>), grid, dim3(256), 0, s, a);
  else if (w_dtype == DIHIP_F32) hipLaunchKernelGGL((linear_tile_kernel<DIHIP_BF16, DIHIP_F32>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((linear_tile_kernel<DIHIP_BF16, DIHIP_BF16>), grid, dim3(256), 0, s, a);
  return launch_status();
}

extern "C" int dihip_linear(void* stream, const void* x, int x_dtype, long ldx, long x_gstride, int x_groups, const void* w,
                            int w_dtype, const void* bias, void* y, int y_dtype, long ldy, long y_gstride, const float* mul,
                            long ldm, int T, int N, int K, int groups, int act, int act_lo, int act_hi, int math) {
  return linear_impl(stream, x, x_dtype, ldx, x_gstride, x_groups, w, w_dtype, bias, y, y_dtype, ldy, y_gstride, mul, ldm, T, N, K, groups,
                     act, act_lo, act_hi, math, nullptr, nullptr, 0);
}

extern "C" int dihip_linear_segmented(void* stream, const void* x, int x_dtype, long ldx, const void* w, int w_dtype, const void* bias,
                                      void* y, int y_dtype, long ldy, int R, int N, int K, int groups, const int32_t* seg,
                                      const int32_t* row_map, int seg_max_rows, int act, int math) {
  DIHIP_REQUIRE(seg && seg_max_rows >= 0, DIHIP_PARAM_ERROR, "linear_segmented: no segment table");
  if (seg_max_rows == 0) return DIHIP_SUCCESS;
  return linear_impl(stream, x, x_dtype, ldx, 0, 1, w, w_dtype, bias, y, y_dtype, ldy, 0, nullptr, 0, R, N, K, groups, act, 0,
                     act ? groups * N : 0, math, seg, row_map, seg_max_rows);
}
