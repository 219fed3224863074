// seq_gla.hip -- gated linear attention with a matrix state per head, everything in f32:
//   per head and row   alpha = sigmoid(z)^(1/tau)  (as exp(log sigmoid(z) / tau)),   S <- diag(alpha) S + k v^T,   o = S^T (q * q_scale)
// S [D, DV] lives per state slot and is carried from portion to portion.  The columns of S are independent, so a workgroup
// owns 64 columns of one head: thread (slice, column) keeps D / 4 rows of its column in registers, rows of the step are
// staged eight at a time in LDS (decays computed once per row and channel), partial dot products of the four slices are
// summed in a fixed order.  Long portions are cut into chunks of 64 rows that run side by side: (1) every chunk composes
// its rows from S = 0 -> (product of its decays, the state it would end in), (2) the states the chunks really start from
// are carried over the chunks, (3) every chunk runs its rows from that state and writes the outputs.
// Beside it: the unit-RMS norm of every head's output times a multiplier (the output gate).
#include "seq_common.h"

namespace dihip {
namespace {

constexpr int GLA_CHUNK = 64, GLA_RB = 8;

struct GlaArgs {
  float* out; long ldo;
  const float* q; long ldq; const float* k; long ldk; const float* v; long ldv; const float* z; long ldz;
  float q_scale, inv_tau;
  float* state;                       // [slots][H][D][DV]
  const int32_t* ent_slot; const int32_t* ent_row0; const int32_t* ent_count;
  int H, D, DV;
  float* ws; int max_chunks;          // ws: [E][max_chunks][H] records of D * DV (state) + D (decay product) floats
};

__device__ __forceinline__ float log_sigmoid(float z) { return -(log1pf(expf(-fabsf(z))) + fmaxf(-z, 0.f)); }

// PASS 0: the whole portion from the slot's state (writes outputs and the state).  PASS 1 / 3: see above.
template <int DPT, int PASS>
__global__ __launch_bounds__(256) void gla_kernel(GlaArgs a) {
  __shared__ __attribute__((aligned(16))) float qs[GLA_RB][4 * DPT];
  __shared__ __attribute__((aligned(16))) float ks[GLA_RB][4 * DPT];
  __shared__ __attribute__((aligned(16))) float as[GLA_RB][4 * DPT];
  __shared__ float vs[GLA_RB][64];
  __shared__ float part[GLA_RB][4][64];
  const int tid = threadIdx.x, lane = tid & 63, sl = tid >> 6;
  const int D = a.D, DV = a.DV, H = a.H;
  const int cbs = (DV + 63) / 64;
  const int ch = blockIdx.x, h = blockIdx.y / cbs, cb = blockIdx.y - h * cbs, e = blockIdx.z;
  const int cnt = a.ent_count[e], row0 = a.ent_row0[e];
  const int lo = PASS == 0 ? 0 : ch * GLA_CHUNK;
  if (lo >= cnt) return;
  const int n = PASS == 0 ? cnt : min(GLA_CHUNK, cnt - lo);
  const int j = cb * 64 + lane;
  const bool col = j < DV;
  const size_t rec = (size_t)D * DV + D;
  float* wrec = PASS == 0 ? nullptr : a.ws + (((size_t)e * a.max_chunks + ch) * H + h) * rec;
  float* sp = a.state + ((size_t)a.ent_slot[e] * H + h) * D * DV;
  float S[DPT];
#pragma unroll
  for (int ii = 0; ii < DPT; ++ii) {
    const int i = sl * DPT + ii;
    S[ii] = 0.f;
    if (PASS != 1 && col && i < D) S[ii] = PASS == 0 ? sp[(size_t)i * DV + j] : wrec[(size_t)i * DV + j];
  }
  float Ap[DPT];   // PASS 1: product of the decays of the thread's channels
#pragma unroll
  for (int ii = 0; ii < DPT; ++ii) Ap[ii] = 1.f;
  for (int b0 = 0; b0 < n; b0 += GLA_RB) {
    const int nb = min(GLA_RB, n - b0);
    __syncthreads();   // the batch before is no longer read
    for (int u = tid; u < GLA_RB * 4 * DPT; u += 256) {
      const int r = u / (4 * DPT), i = u - r * (4 * DPT);
      float qv = 0.f, kv = 0.f, av = 1.f;
      if (r < nb && i < D) {
        const size_t t = (size_t)(row0 + lo + b0 + r);
        const size_t c = (size_t)h * D + i;
        if (PASS != 1) qv = a.q[t * a.ldq + c] * a.q_scale;
        kv = a.k[t * a.ldk + c];
        av = expf(log_sigmoid(a.z[t * a.ldz + c]) * a.inv_tau);
      }
      qs[r][i] = qv; ks[r][i] = kv; as[r][i] = av;
    }
    for (int u = tid; u < GLA_RB * 64; u += 256) {
      const int r = u >> 6, c = u & 63;
      vs[r][c] = (r < nb && cb * 64 + c < DV) ? a.v[(size_t)(row0 + lo + b0 + r) * a.ldv + (size_t)h * DV + cb * 64 + c] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < GLA_RB; ++r) {
      if (r < nb) {
        const float vj = vs[r][lane];
        float po = 0.f;
#pragma unroll
        for (int i4 = 0; i4 < DPT; i4 += 4) {
          const f32x4_t a4 = *reinterpret_cast<const f32x4_t*>(&as[r][sl * DPT + i4]);
          const f32x4_t k4 = *reinterpret_cast<const f32x4_t*>(&ks[r][sl * DPT + i4]);
          const f32x4_t q4 = *reinterpret_cast<const f32x4_t*>(&qs[r][sl * DPT + i4]);
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            S[i4 + x] = __builtin_fmaf(a4[x], S[i4 + x], k4[x] * vj);
            if (PASS == 1) Ap[i4 + x] *= a4[x];
            else po = __builtin_fmaf(S[i4 + x], q4[x], po);
          }
        }
        if (PASS != 1) part[r][sl][lane] = po;
      }
    }
    if (PASS != 1) {
      __syncthreads();
      for (int u = tid; u < nb * 64; u += 256) {
        const int r = u >> 6, c = u & 63;
        if (cb * 64 + c < DV)
          a.out[(size_t)(row0 + lo + b0 + r) * a.ldo + (size_t)h * DV + cb * 64 + c] = (part[r][0][c] + part[r][1][c]) + (part[r][2][c] + part[r][3][c]);
      }
    }
  }
  if (PASS == 1) {
#pragma unroll
    for (int ii = 0; ii < DPT; ++ii) {
      const int i = sl * DPT + ii;
      if (i < D) {
        if (col) wrec[(size_t)i * DV + j] = S[ii];
        if (cb == 0 && lane == 0) wrec[(size_t)D * DV + i] = Ap[ii];
      }
    }
  } else if (PASS == 0 || lo + n == cnt) {
#pragma unroll
    for (int ii = 0; ii < DPT; ++ii) {
      const int i = sl * DPT + ii;
      if (col && i < D) sp[(size_t)i * DV + j] = S[ii];
    }
  }
}

// pass 2: per state element, chunks in order: record <- the state the chunk starts from;  S <- decay product * S + record
__global__ __launch_bounds__(256) void gla_carry_kernel(GlaArgs a) {
  const int e = blockIdx.z, h = blockIdx.y;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.D * a.DV) return;
  const int i = idx / a.DV;
  const int chunks = (a.ent_count[e] + GLA_CHUNK - 1) / GLA_CHUNK;
  const size_t rec = (size_t)a.D * a.DV + a.D;
  float S = a.state[((size_t)a.ent_slot[e] * a.H + h) * a.D * a.DV + idx];
  for (int ch = 0; ch < chunks; ++ch) {
    float* wrec = a.ws + (((size_t)e * a.max_chunks + ch) * a.H + h) * rec;
    const float U = wrec[idx], A = wrec[(size_t)a.D * a.DV + i];
    wrec[idx] = S;
    S = __builtin_fmaf(A, S, U);
  }
}

template <int WT>
__global__ __launch_bounds__(256) void head_rmsnorm_mul_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ x, long ldx,
                                                               const void* __restrict__ gamma, float eps, const float* __restrict__ mul,
                                                               long ldm, int H, int DV) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int h = wave; h < H; h += 4) {
    const float* xr = x + (size_t)t * ldx + (size_t)h * DV;
    float ss = 0.f;
    for (int d = lane; d < DV; d += 64) ss = __builtin_fmaf(xr[d], xr[d], ss);
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)DV + eps);
    for (int d = lane; d < DV; d += 64) {
      float v = xr[d] * inv * load_ft<WT>(gamma, d);
      if (mul) v *= mul[(size_t)t * ldm + (size_t)h * DV + d];
      st_any(y, (size_t)t * ldy + (size_t)h * DV + d, ydt, v);
    }
  }
}

}  // namespace
}  // namespace dihip

using namespace dihip;

extern "C" {

size_t dihip_gla_chunked_workspace_bytes(int E, int max_count, int H, int D, int DV) {
  return (size_t)E * ((max_count + GLA_CHUNK - 1) / GLA_CHUNK) * H * ((size_t)D * DV + D) * sizeof(float);
}

int dihip_gla(void* stream, float* out, long ldo, const float* q, long ldq, const float* k, long ldk, const float* v, long ldv,
              const float* z, long ldz, float q_scale, float tau, float* state, const int32_t* ent_slot, const int32_t* ent_row0,
              const int32_t* ent_count, int E, int max_count, int H, int D, int DV, int chunked, void* ws, size_t ws_bytes) {
  DIHIP_REQUIRE(E >= 0 && max_count >= 0 && H > 0 && D > 0 && DV > 0 && out && q && k && v && z && state && ent_slot && ent_row0 && ent_count &&
                    ldo >= (long)H * DV && ldq >= (long)H * D && ldk >= (long)H * D && ldz >= (long)H * D && ldv >= (long)H * DV && tau > 0.f,
                DIHIP_PARAM_ERROR, "gla: bad argument");
  DIHIP_REQUIRE(D <= 256, DIHIP_EXCEED_LIMIT_ERROR, "gla: more than 256 key channels per head (%d)", D);
  const int cbs = (DV + 63) / 64;
  DIHIP_REQUIRE((long)H * cbs <= 65535 && E <= 65535, DIHIP_PARAM_ERROR, "gla: too many heads or portions for one launch");
  DIHIP_REQUIRE(!chunked || (ws && ws_bytes >= dihip_gla_chunked_workspace_bytes(E, max_count, H, D, DV)), DIHIP_PARAM_ERROR,
                "gla: workspace too small");
  if (E == 0 || max_count == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int chunks = chunked ? (max_count + GLA_CHUNK - 1) / GLA_CHUNK : 1;
  GlaArgs a{out, ldo, q, ldq, k, ldk, v, ldv, z, ldz, q_scale, 1.f / tau, state, ent_slot, ent_row0, ent_count, H, D, DV, (float*)ws, chunks};
  const dim3 grid(chunks, H * cbs, E);
  auto go = [&](auto dpt) {
    constexpr int DPT = decltype(dpt)::value;
    if (!chunked) {
      hipLaunchKernelGGL((gla_kernel<DPT, 0>), grid, dim3(256), 0, s, a);
    } else {
      hipLaunchKernelGGL((gla_kernel<DPT, 1>), grid, dim3(256), 0, s, a);
      hipLaunchKernelGGL(gla_carry_kernel, dim3((D * DV + 255) / 256, H, E), dim3(256), 0, s, a);
      hipLaunchKernelGGL((gla_kernel<DPT, 3>), grid, dim3(256), 0, s, a);
    }
  };
  if (D <= 64) go(std::integral_constant<int, 16>{});
  else if (D <= 128) go(std::integral_constant<int, 32>{});
  else go(std::integral_constant<int, 64>{});
  return launch_status();
}

int dihip_head_rmsnorm_mul(void* stream, void* y, int y_dtype, long ldy, const float* x, long ldx, const void* gamma, int w_dtype,
                           float eps, const float* mul, long ldm, int T, int H, int DV) {
  DIHIP_REQUIRE(T >= 0 && H > 0 && DV > 0 && y && x && gamma && ldy >= (long)H * DV && ldx >= (long)H * DV && (!mul || ldm >= (long)H * DV) &&
                    seq_dtype_ok(y_dtype) && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR, "head_rmsnorm_mul: bad argument");
  if (T == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (w_dtype == DIHIP_F32) hipLaunchKernelGGL(head_rmsnorm_mul_kernel<DIHIP_F32>, dim3(T), dim3(256), 0, s, y, y_dtype, ldy, x, ldx, gamma, eps, mul, ldm, H, DV);
  else hipLaunchKernelGGL(head_rmsnorm_mul_kernel<DIHIP_BF16>, dim3(T), dim3(256), 0, s, y, y_dtype, ldy, x, ldx, gamma, eps, mul, ldm, H, DV);
  return launch_status();
}

}  // extern "C"
