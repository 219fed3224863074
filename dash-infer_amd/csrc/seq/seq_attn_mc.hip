// seq_attn_mc.hip -- windowed sink-softmax attention over the paged latent cache on the matrix cores (bf16 cache).
//
// All heads of a sequence share the cached latent rows C [keys, R]: they are keys AND values.  A workgroup owns 64
// consecutive (row, head) pairs of one portion -- 16 per wave -- and walks the key tiles of 32 cached rows its pairs can
// see.  Per tile: S^T = C . Q^T (A = the tile's rows as they lie in LDS, B = the wave's query fragments, held in registers
// for the whole walk), mask + running softmax on the accumulator lanes (a pair's 32 scores sit in the four 16-lane groups
// of one lane column: permlane swaps reduce them), then O^T += C^T . P^T with P taken straight from those lanes and
// C^T read from the same LDS tile through the transposing LDS read.  The next tile's rows are in flight meanwhile.
// The key walk can be split over gridDim.z workgroups (few rows: decoding); the partial (maximum, denominator, sums)
// records are merged by a second launch.  The sink joins split 0 as the running softmax's start (maximum = sink,
// denominator = 1).
#include "seq_common.h"

namespace dihip {
namespace {

struct McArgs {
  float* out; long ldo;
  const float* q; long ldq;
  void* const* spans; int span_stride, span_len;
  const void* sink; int wdt;
  const int32_t* tok_pos; const int32_t* ent_slot; const int32_t* ent_row0; const int32_t* ent_count;
  int H, R, window; float scale;
  float* ws; int rows_total;
};

__device__ __forceinline__ f32x4_t mfma_bf16x(const u32x4_t& a, const u32x4_t& b, const f32x4_t& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

template <int RMAX>
__global__ __launch_bounds__(256) void latent_attn_mc_kernel(McArgs a) {
  constexpr int KS = RMAX / 32, DT = RMAX / 16, UN = RMAX / 64;
  constexpr bool PREFETCH = RMAX <= 256;  // the widest rows leave no registers for a tile in flight
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int e = blockIdx.y, split = blockIdx.z, nsplit = gridDim.z;
  const int H = a.H, R = a.R;
  const int cnt = a.ent_count[e], row0 = a.ent_row0[e];
  const int nrows = cnt * H, r0 = blockIdx.x * 64;
  if (r0 >= nrows) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, ni = lane & 15, kb = lane >> 4;
  const int pitch = R + 8, pitchb = pitch * 2;
  const int pos0 = a.tok_pos[row0];
  const int myrow = r0 + wave * 16 + ni;
  const bool row_ok = myrow < nrows;
  const int rr = row_ok ? myrow : nrows - 1;
  const int tq = rr / H, h = rr - tq * H, p = pos0 + tq;
  const int p_lo = pos0 + r0 / H, p_hi = pos0 + min(r0 + 63, nrows - 1) / H;
  const int k_begin = a.window > 0 ? max(0, p_lo - a.window + 1) : 0;
  const int tile_lo = k_begin >> 5, tile_hi = p_hi >> 5;
  const int per = (tile_hi - tile_lo + nsplit) / nsplit;
  const int my_lo = tile_lo + split * per, my_hi = min(tile_hi, my_lo + per - 1);

  u32x4_t qf[KS];
  {
    const float* qrow = a.q + (size_t)(row0 + tq) * a.ldq + (size_t)h * R;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = u32x4_t{0u, 0u, 0u, 0u};
      if (ks * 32 < R) {
        const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(qrow + ks * 32 + kb * 8);
        const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(qrow + ks * 32 + kb * 8 + 4);
        qf[ks] = u32x4_t{pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]), pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3])};
      }
    }
  }
  const bool with_sink = a.sink != nullptr && split == 0;
  float m = with_sink ? ld_any(a.sink, h, a.wdt) : -1e30f;
  float l = with_sink ? 1.f : 0.f;
  const f32x4_t z4 = {0.f, 0.f, 0.f, 0.f};
  f32x4_t oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) oacc[t] = z4;

  // the span pointers of the walk, staged once: a tile's loads then depend on nothing that is still in flight
  __shared__ const char* tabs[128];
  void* const* gtab = a.spans + (size_t)a.ent_slot[e] * a.span_stride;
  const int span_lo = (my_lo * 32) / a.span_len;
  for (int i = tid; i < 128; i += 256) {
    const int sp = span_lo + i;
    tabs[i] = (sp * a.span_len <= p_hi) ? (const char*)gtab[sp] : nullptr;
  }
  __syncthreads();
  // a thread's 16-byte units of a tile: (key inside the tile, column) fixed for the whole walk -- the divisions are done once.
  // A tile of 32 keys lies inside one span (span_len % 32 == 0): its span and offset are wave-uniform.
  const int upr = R >> 3;  // 16-byte units per cached row
  int goff[UN], loff[UN];
#pragma unroll
  for (int j = 0; j < UN; ++j) {
    const int u = tid + 256 * j, kin = u / upr, c8 = u - kin * upr;
    goff[j] = kin < 32 ? (kin * R + c8 * 8) * 2 : -1;
    loff[j] = kin * pitchb + c8 * 16;
  }
  u32x4_t pre[UN];
  auto fetch = [&](int tile) {
    const int key0 = tile * 32, sp = key0 / a.span_len;
    const char* sb = (sp - span_lo < 128 ? tabs[sp - span_lo] : (const char*)gtab[sp]) + (size_t)(key0 - sp * a.span_len) * R * 2;
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      pre[j] = u32x4_t{0u, 0u, 0u, 0u};
      if (goff[j] >= 0) pre[j] = gload<u32x4_t>(sb + goff[j]);
    }
  };
  if (PREFETCH && my_lo <= my_hi) fetch(my_lo);
  for (int tile = my_lo; tile <= my_hi; ++tile) {
    if (!PREFETCH) fetch(tile);
#pragma unroll
    for (int j = 0; j < UN; ++j)
      if (goff[j] >= 0) *reinterpret_cast<u32x4_t*>(smem + loff[j]) = pre[j];
    __syncthreads();
    if (PREFETCH && tile + 1 <= my_hi) fetch(tile + 1);
    f32x4_t sacc[2] = {z4, z4};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks * 32 < R) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          const u32x4_t kf = *reinterpret_cast<const u32x4_t*>(smem + (nt * 16 + ni) * pitchb + (ks * 32 + kb * 8) * 2);
          sacc[nt] = mfma_bf16x(kf, qf[ks], sacc[nt]);
        }
      }
    }
    float sv[2][4], mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = tile * 32 + nt * 16 + kb * 4 + r;
        const bool vis = key <= p && (a.window <= 0 || key > p - a.window);
        sv[nt][r] = vis ? sacc[nt][r] * a.scale : -INFINITY;
        mx = fmaxf(mx, sv[nt][r]);
      }
    mx = rows_max(mx);
    const float mn = fmaxf(m, mx);
    const float corr = __expf(m - mn);
    m = mn;
    float psum = 0.f, ev[2][4];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        ev[nt][r] = __expf(sv[nt][r] - mn);
        psum += ev[nt][r];
      }
    l = l * corr + rows_sum(psum);
    const u32x4_t pf = {pack_bf16x2(ev[0][0], ev[0][1]), pack_bf16x2(ev[0][2], ev[0][3]), pack_bf16x2(ev[1][0], ev[1][1]),
                        pack_bf16x2(ev[1][2], ev[1][3])};
    if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0ull) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) oacc[t][r] *= corr;
    }
    const unsigned char* tr0 = smem + (kb * 4 + (ni >> 2)) * pitchb + (ni & 3) * 8;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      if (t * 16 < R) {
        const u32x2_t lo2 = lds_read_tr16(tr0 + t * 32);
        const u32x2_t hi2 = lds_read_tr16(tr0 + t * 32 + 16 * pitchb);
        const u32x4_t vf = {lo2[0], lo2[1], hi2[0], hi2[1]};
        oacc[t] = mfma_bf16x(vf, pf, oacc[t]);
      }
    }
    __syncthreads();
  }
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
  if (!row_ok) return;
  if (nsplit == 1) {
    const float inv = 1.f / l;
    float* o = a.out + (size_t)(row0 + tq) * a.ldo + (size_t)h * R + kb * 4;
#pragma unroll
    for (int t = 0; t < DT; ++t)
      if (t * 16 < R) *reinterpret_cast<f32x4_t*>(o + t * 16) = f32x4_t{oacc[t][0] * inv, oacc[t][1] * inv, oacc[t][2] * inv, oacc[t][3] * inv};
  } else {
    float* o = a.ws + ((size_t)split * a.rows_total + (size_t)(row0 + tq) * H + h) * (R + 4);
#pragma unroll
    for (int t = 0; t < DT; ++t)
      if (t * 16 < R) *reinterpret_cast<f32x4_t*>(o + t * 16 + kb * 4) = oacc[t];
    if (kb == 0) { o[R] = m; o[R + 1] = l; }
  }
}

__global__ __launch_bounds__(256) void latent_attn_merge_kernel(float* __restrict__ out, long ldo, const float* __restrict__ ws, int nsplit,
                                                                int rows_total, int H, int R) {
  __shared__ float wgt[1024];
  __shared__ float red[4];
  const int g = blockIdx.x, t = g / H, h = g - t * H;
  const size_t rec = (size_t)R + 4, stride = (size_t)rows_total * rec;
  const float* base = ws + (size_t)g * rec;
  float mloc[4], lloc[4], mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int s = threadIdx.x + i * 256;
    mloc[i] = s < nsplit ? base[s * stride + R] : -INFINITY;
    lloc[i] = s < nsplit ? base[s * stride + R + 1] : 0.f;
    mx = fmaxf(mx, mloc[i]);
  }
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float den = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int s = threadIdx.x + i * 256;
    const float w = s < nsplit ? expf(mloc[i] - mx) : 0.f;
    if (s < nsplit) wgt[s] = w;
    den = __builtin_fmaf(w, lloc[i], den);
  }
  den = block256_sum(den, red);      // (its barriers publish wgt)
  const float inv = 1.f / den;
  for (int r = threadIdx.x; r < R; r += 256) {
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < nsplit; ++s) acc = __builtin_fmaf(wgt[s], base[s * stride + r], acc);
    out[(size_t)t * ldo + (size_t)h * R + r] = acc * inv;
  }
}

}  // namespace
}  // namespace dihip

using namespace dihip;

extern "C" {

int dihip_latent_window_attn_mc_supported(int R, int span_len, int cache_dtype) {
  return cache_dtype == DIHIP_BF16 && R % 32 == 0 && R >= 32 && R <= 512 && span_len % 32 == 0;
}

size_t dihip_latent_window_attn_mc_workspace_bytes(int T, int H, int R, int nsplit) {
  return nsplit > 1 ? (size_t)nsplit * T * H * (R + 4) * sizeof(float) : 0;
}

int dihip_latent_window_attn_mc(void* stream, float* out, long ldo, const float* q, long ldq, void* const* spans, int span_stride,
                                int span_len, const void* sink, int w_dtype, const int32_t* tok_pos, const int32_t* ent_slot,
                                const int32_t* ent_row0, const int32_t* ent_count, int E, int max_count, int T, int H, int R, int window,
                                float scale, int nsplit, void* ws, size_t ws_bytes) {
  DIHIP_REQUIRE(dihip_latent_window_attn_mc_supported(R, span_len, DIHIP_BF16), DIHIP_PARAM_ERROR,
                "latent_window_attn_mc: R %d (a multiple of 32 up to 512) / span_len %d (a multiple of 32) not served", R, span_len);
  DIHIP_REQUIRE(E >= 0 && T >= 0 && H > 0 && max_count >= 0 && out && q && spans && tok_pos && ent_slot && ent_row0 && ent_count &&
                    span_stride > 0 && ldo >= (long)H * R && ldq >= (long)H * R && ldo % 4 == 0 && ldq % 4 == 0 && seq_dtype_ok(w_dtype),
                DIHIP_PARAM_ERROR, "latent_window_attn_mc: bad argument");
  DIHIP_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15u) == 0 && (reinterpret_cast<uintptr_t>(q) & 15u) == 0, DIHIP_PARAM_ERROR,
                "latent_window_attn_mc: q / out must be 16-byte aligned");
  DIHIP_REQUIRE(nsplit >= 1 && nsplit <= 1024 && E <= 65535, DIHIP_PARAM_ERROR, "latent_window_attn_mc: bad split / portion count");
  DIHIP_REQUIRE(ws_bytes >= dihip_latent_window_attn_mc_workspace_bytes(T, H, R, nsplit) && (nsplit == 1 || ws), DIHIP_PARAM_ERROR,
                "latent_window_attn_mc: workspace too small");
  if (E == 0 || max_count == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  McArgs a{out, ldo, q, ldq, spans, span_stride, span_len, sink, w_dtype, tok_pos, ent_slot, ent_row0, ent_count, H, R, window, scale,
           (float*)ws, T * H};
  const dim3 grid((unsigned)(((long)max_count * H + 63) / 64), E, nsplit);
  const size_t lds = (size_t)32 * (R + 8) * 2;
  if (R <= 64) hipLaunchKernelGGL(latent_attn_mc_kernel<64>, grid, dim3(256), lds, s, a);
  else if (R <= 128) hipLaunchKernelGGL(latent_attn_mc_kernel<128>, grid, dim3(256), lds, s, a);
  else if (R <= 256) hipLaunchKernelGGL(latent_attn_mc_kernel<256>, grid, dim3(256), lds, s, a);
  else hipLaunchKernelGGL(latent_attn_mc_kernel<512>, grid, dim3(256), lds, s, a);
  if (nsplit > 1) hipLaunchKernelGGL(latent_attn_merge_kernel, dim3(T * H), dim3(256), 0, s, out, ldo, (const float*)ws, nsplit, T * H, H, R);
  return launch_status();
}

}  // extern "C"
