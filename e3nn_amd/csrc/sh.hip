// Spherical harmonics kernels (gfx950).
//
// Fast path, l = 0..LMAX with LMAX <= 3: closed-form polynomials
// (reference e3nn/o3/_spherical_harmonics.py:194-226).  One wavefront owns a tile of 64
// vectors: the 768-byte input tile is fetched with 48 dwordx4 loads and redistributed
// through LDS, every lane evaluates one vector, and the 64 x NC output tile goes back
// through LDS so that each store instruction writes 1 KiB of consecutive addresses.
// The kernel is pure streaming: 12 B in + 4 NC B out per vector.
//
// Generic path, any list of l <= 12: the recurrence the reference's generator used
// (e3nn/o3/_spherical_harmonics_generator.py:57-65), driven by a sparse table of
// wigner_3j(l+1, 1, l) in constant memory; per-lane values live in LDS columns.
#include <hip/hip_runtime.h>

#include <cmath>
#include <mutex>
#include <vector>

#include "e3x_internal.h"

namespace {

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;

// Orders this wavefront's LDS writes before its later LDS reads (no other wave shares
// the buffer, so no workgroup barrier is needed and loop trip counts may differ per wave).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int LMAX>
__device__ __forceinline__ void sh_poly(float x, float y, float z, float (&o)[(LMAX + 1) * (LMAX + 1)],
                                        const float (&scale)[4]) {
  o[0] = scale[0];
  if constexpr (LMAX >= 1) {
    const float c = 1.7320508075688772f * scale[1];
    o[1] = c * x;
    o[2] = c * y;
    o[3] = c * z;
  }
  if constexpr (LMAX >= 2) {
    const float r15 = 3.872983346207417f, r5 = 2.23606797749979f;
    const float y2 = y * y, s = x * x + z * z;
    const float a20 = r15 * x * z;
    const float a24 = 0.5f * r15 * (z * z - x * x);
    o[4] = scale[2] * a20;
    o[5] = scale[2] * (r15 * x * y);
    o[6] = scale[2] * (r5 * (y2 - 0.5f * s));
    o[7] = scale[2] * (r15 * y * z);
    o[8] = scale[2] * a24;
    if constexpr (LMAX >= 3) {
      const float r7 = 2.6457513110645907f;
      const float c0 = 1.0801234497346435f;  // sqrt(42)/6
      const float c2 = 1.6201851746019651f;  // sqrt(168)/8
      const float t = 4.0f * y2 - s;
      o[9] = scale[3] * (c0 * (a20 * z + a24 * x));
      o[10] = scale[3] * (r7 * a20 * y);
      o[11] = scale[3] * (c2 * t * x);
      o[12] = scale[3] * (0.5f * r7 * y * (2.0f * y2 - 3.0f * s));
      o[13] = scale[3] * (c2 * z * t);
      o[14] = scale[3] * (r7 * a24 * y);
      o[15] = scale[3] * (c0 * (a24 * z - a20 * x));
    }
  }
}

struct Scale4 {
  float s[4];
};

template <int LMAX, bool NORMALIZE>
__global__ __launch_bounds__(kWave* kWavesPerBlock) void sh_tile_kernel(const float* __restrict__ xyz,
                                                                       float* __restrict__ out, long long n,
                                                                       Scale4 sc) {
  constexpr int NC = (LMAX + 1) * (LMAX + 1);
  constexpr int LD = NC | 1;  // odd LDS row stride: conflict-free column access
  __shared__ float s_in[kWavesPerBlock][kWave * 3];
  __shared__ float s_out[kWavesPerBlock][kWave * LD];
  const int lane = threadIdx.x & (kWave - 1);
  const int wv = threadIdx.x / kWave;
  const long long n_tiles = (n + kWave - 1) / kWave;
  const float scale[4] = {sc.s[0], sc.s[1], sc.s[2], sc.s[3]};

  for (long long tile = (long long)blockIdx.x * kWavesPerBlock + wv; tile < n_tiles;
       tile += (long long)gridDim.x * kWavesPerBlock) {
    const long long v0 = tile * kWave;
    const int nv = (int)min((long long)kWave, n - v0);
    float x, y, z;
    if (nv == kWave) {
      if (lane < 48) {
        const float4 q = reinterpret_cast<const float4*>(xyz + v0 * 3)[lane];
        reinterpret_cast<float4*>(s_in[wv])[lane] = q;
      }
      wave_lds_sync();
      x = s_in[wv][lane * 3 + 0];
      y = s_in[wv][lane * 3 + 1];
      z = s_in[wv][lane * 3 + 2];
    } else {
      x = y = z = 0.0f;
      if (lane < nv) {
        x = xyz[(v0 + lane) * 3 + 0];
        y = xyz[(v0 + lane) * 3 + 1];
        z = xyz[(v0 + lane) * 3 + 2];
      }
    }
    if constexpr (NORMALIZE) {
      // x / max(|x|, 1e-12): torch.nn.functional.normalize (reference :96)
      const float nrm = sqrtf(x * x + y * y + z * z);
      const float inv = 1.0f / fmaxf(nrm, 1e-12f);
      x *= inv;
      y *= inv;
      z *= inv;
    }
    float o[NC];
    sh_poly<LMAX>(x, y, z, o, scale);
#pragma unroll
    for (int c = 0; c < NC; ++c) s_out[wv][lane * LD + c] = o[c];
    wave_lds_sync();
    float* dst = out + v0 * NC;
    if (nv == kWave) {
      constexpr int NQ = kWave * NC / 4;  // float4 per tile
#pragma unroll
      for (int q0 = 0; q0 < NQ; q0 += kWave) {
        const int q = q0 + lane;
        if (NQ % kWave == 0 || q < NQ) {
          float4 v;
          float* pv = reinterpret_cast<float*>(&v);
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int e = q * 4 + t;
            pv[t] = s_out[wv][(e / NC) * LD + (e % NC)];
          }
          reinterpret_cast<float4*>(dst)[q] = v;
        }
      }
    } else {
      for (int e = lane; e < nv * NC; e += kWave) dst[e] = s_out[wv][(e / NC) * LD + (e % NC)];
    }
    wave_lds_sync();
  }
}

// ---------------------------------------------------------------- backward, l <= 3
// Forward-mode duals: every polynomial carries its gradient with respect to the (normalised)
// input, so the derivative code is the forward code (no hand-derived formulas to get wrong).
struct Dual {
  float v, dx, dy, dz;
  static __device__ __forceinline__ Dual constant(float c) { return {c, 0.f, 0.f, 0.f}; }
};
__device__ __forceinline__ Dual operator+(Dual a, Dual b) { return {a.v + b.v, a.dx + b.dx, a.dy + b.dy, a.dz + b.dz}; }
__device__ __forceinline__ Dual operator-(Dual a, Dual b) { return {a.v - b.v, a.dx - b.dx, a.dy - b.dy, a.dz - b.dz}; }
__device__ __forceinline__ Dual operator*(Dual a, Dual b) {
  return {a.v * b.v, fmaf(a.v, b.dx, a.dx * b.v), fmaf(a.v, b.dy, a.dy * b.v), fmaf(a.v, b.dz, a.dz * b.v)};
}
__device__ __forceinline__ Dual operator*(float c, Dual a) { return {c * a.v, c * a.dx, c * a.dy, c * a.dz}; }

// Second order: a value with its gradient d[i] = d/dx_i, its derivative a = d/dt along one fixed direction, and the
// gradient of that directional derivative, ad[i] = d^2 / (dt dx_i) -- what the derivative of a backward pass needs
// (the Hessian applied to one vector), again with the forward code as derivative code.
struct Dual2 {
  float v, d[3], a, ad[3];
  static __device__ __forceinline__ Dual2 constant(float c) { return {c, {0.f, 0.f, 0.f}, 0.f, {0.f, 0.f, 0.f}}; }
};
__device__ __forceinline__ Dual2 operator+(Dual2 p, Dual2 q) {
  return {p.v + q.v, {p.d[0] + q.d[0], p.d[1] + q.d[1], p.d[2] + q.d[2]}, p.a + q.a, {p.ad[0] + q.ad[0], p.ad[1] + q.ad[1], p.ad[2] + q.ad[2]}};
}
__device__ __forceinline__ Dual2 operator-(Dual2 p, Dual2 q) {
  return {p.v - q.v, {p.d[0] - q.d[0], p.d[1] - q.d[1], p.d[2] - q.d[2]}, p.a - q.a, {p.ad[0] - q.ad[0], p.ad[1] - q.ad[1], p.ad[2] - q.ad[2]}};
}
__device__ __forceinline__ Dual2 operator*(Dual2 p, Dual2 q) {
  Dual2 r;
  r.v = p.v * q.v;
  r.a = fmaf(p.a, q.v, p.v * q.a);
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    r.d[i] = fmaf(p.d[i], q.v, p.v * q.d[i]);
    r.ad[i] = fmaf(p.ad[i], q.v, fmaf(p.d[i], q.a, fmaf(p.a, q.d[i], p.v * q.ad[i])));
  }
  return r;
}
__device__ __forceinline__ Dual2 operator*(float c, Dual2 p) {
  return {c * p.v, {c * p.d[0], c * p.d[1], c * p.d[2]}, c * p.a, {c * p.ad[0], c * p.ad[1], c * p.ad[2]}};
}
// f(p) for a scalar function with f(p.v) = f0, f'(p.v) = f1, f''(p.v) = f2
__device__ __forceinline__ Dual2 chain(Dual2 p, float f0, float f1, float f2) {
  Dual2 r;
  r.v = f0;
  r.a = f1 * p.a;
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    r.d[i] = f1 * p.d[i];
    r.ad[i] = fmaf(f2 * p.a, p.d[i], f1 * p.ad[i]);
  }
  return r;
}

template <int LMAX, class D>
__device__ __forceinline__ void sh_poly_dual(D x, D y, D z, D (&o)[(LMAX + 1) * (LMAX + 1)]) {
  o[0] = D::constant(1.f);
  if constexpr (LMAX >= 1) {
    const float c = 1.7320508075688772f;
    o[1] = c * x;
    o[2] = c * y;
    o[3] = c * z;
  }
  if constexpr (LMAX >= 2) {
    const float r15 = 3.872983346207417f, r5 = 2.23606797749979f;
    const D y2 = y * y, s = x * x + z * z;
    const D a20 = r15 * (x * z);
    const D a24 = (0.5f * r15) * (z * z - x * x);
    o[4] = a20;
    o[5] = r15 * (x * y);
    o[6] = r5 * (y2 - 0.5f * s);
    o[7] = r15 * (y * z);
    o[8] = a24;
    if constexpr (LMAX >= 3) {
      const float r7 = 2.6457513110645907f, c0 = 1.0801234497346435f, c2 = 1.6201851746019651f;
      const D t = 4.0f * y2 - s;
      o[9] = c0 * (a20 * z + a24 * x);
      o[10] = r7 * (a20 * y);
      o[11] = c2 * (t * x);
      o[12] = (0.5f * r7) * (y * (2.0f * y2 - 3.0f * s));
      o[13] = c2 * (z * t);
      o[14] = r7 * (a24 * y);
      o[15] = c0 * (a24 * z - a20 * x);
    }
  }
}

// The derivative of the backward pass.  With phi(x) = sum_c g_c Y_c(x) the backward pass returns grad phi; for a
// cotangent t[3] on that result this kernel returns d<t, grad phi>/dg_c = (directional derivative of Y_c along t) and
// d<t, grad phi>/dx = (Hessian of phi) t, from one evaluation of the polynomials on Dual2 numbers whose fixed
// direction is t.  The normalisation x / max(|x|, 1e-12) is part of the differentiated function.
template <int LMAX, bool NORMALIZE>
__global__ __launch_bounds__(256) void sh_bwd2_kernel(const float* __restrict__ xyz, const float* __restrict__ gout,
                                                      const float* __restrict__ cot, float* __restrict__ ggout,
                                                      float* __restrict__ gxyz, long long n, Scale4 sc) {
  constexpr int NC = (LMAX + 1) * (LMAX + 1);
  const long long v = (long long)blockIdx.x * 256 + threadIdx.x;
  if (v >= n) return;
  Dual2 p[3];
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    p[i] = Dual2::constant(xyz[v * 3 + i]);
    p[i].d[i] = 1.f;
    p[i].a = cot[v * 3 + i];
  }
  if constexpr (NORMALIZE) {
    const Dual2 s = p[0] * p[0] + p[1] * p[1] + p[2] * p[2];
    const float nrm = sqrtf(s.v);
    Dual2 inv;
    if (nrm < 1e-12f) {
      inv = Dual2::constant(1e12f);  // below the clamp the map is x / 1e-12
    } else {
      const float r = 1.0f / nrm, r2 = r * r;  // s^(-1/2) and its derivatives -1/2 s^(-3/2), 3/4 s^(-5/2)
      inv = chain(s, r, -0.5f * r * r2, 0.75f * r * r2 * r2);
    }
#pragma unroll
    for (int i = 0; i < 3; ++i) p[i] = p[i] * inv;
  }
  Dual2 o[NC];
  sh_poly_dual<LMAX>(p[0], p[1], p[2], o);
  float gx[3] = {0.f, 0.f, 0.f};
  const float* g = gout + v * NC;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int l = c >= 9 ? 3 : (c >= 4 ? 2 : (c >= 1 ? 1 : 0));
    ggout[v * NC + c] = sc.s[l] * o[c].a;
    const float gc = g[c] * sc.s[l];
#pragma unroll
    for (int i = 0; i < 3; ++i) gx[i] = fmaf(gc, o[c].ad[i], gx[i]);
  }
#pragma unroll
  for (int i = 0; i < 3; ++i) gxyz[v * 3 + i] = gx[i];
}

template <int LMAX>
void launch_bwd2(bool normalize, const float* xyz, const float* gout, const float* cot, float* ggout, float* gxyz, long long n,
                 Scale4 sc, hipStream_t st) {
  const long long blocks = (n + 255) / 256;
  if (normalize)
    hipLaunchKernelGGL((sh_bwd2_kernel<LMAX, true>), dim3((unsigned)blocks), dim3(256), 0, st, xyz, gout, cot, ggout, gxyz, n, sc);
  else
    hipLaunchKernelGGL((sh_bwd2_kernel<LMAX, false>), dim3((unsigned)blocks), dim3(256), 0, st, xyz, gout, cot, ggout, gxyz, n, sc);
}

template <int LMAX, bool NORMALIZE>
__global__ __launch_bounds__(256) void sh_bwd_kernel(const float* __restrict__ xyz, const float* __restrict__ gout,
                                                     float* __restrict__ gxyz, long long n, Scale4 sc) {
  constexpr int NC = (LMAX + 1) * (LMAX + 1);
  const long long v = (long long)blockIdx.x * 256 + threadIdx.x;
  if (v >= n) return;
  float x = xyz[v * 3 + 0], y = xyz[v * 3 + 1], z = xyz[v * 3 + 2];
  float inv = 1.0f;
  bool clamped = false;
  if constexpr (NORMALIZE) {
    const float nrm = sqrtf(x * x + y * y + z * z);
    clamped = nrm < 1e-12f;
    inv = 1.0f / fmaxf(nrm, 1e-12f);
    x *= inv;
    y *= inv;
    z *= inv;
  }
  Dual o[NC];
  sh_poly_dual<LMAX>(Dual{x, 1.f, 0.f, 0.f}, Dual{y, 0.f, 1.f, 0.f}, Dual{z, 0.f, 0.f, 1.f}, o);
  float gx = 0.f, gy = 0.f, gz = 0.f;
  const float* g = gout + v * NC;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int l = c >= 9 ? 3 : (c >= 4 ? 2 : (c >= 1 ? 1 : 0));
    const float gc = g[c] * sc.s[l];
    gx = fmaf(gc, o[c].dx, gx);
    gy = fmaf(gc, o[c].dy, gy);
    gz = fmaf(gc, o[c].dz, gz);
  }
  if constexpr (NORMALIZE) {
    // x / max(|x|, eps): for |x| >= eps the Jacobian is (I - u u^T) / |x|, below it is I / eps
    if (!clamped) {
      const float dot = gx * x + gy * y + gz * z;
      gx = (gx - x * dot) * inv;
      gy = (gy - y * dot) * inv;
      gz = (gz - z * dot) * inv;
    } else {
      gx *= inv;
      gy *= inv;
      gz *= inv;
    }
  }
  gxyz[v * 3 + 0] = gx;
  gxyz[v * 3 + 1] = gy;
  gxyz[v * 3 + 2] = gz;
}

template <int LMAX>
void launch_bwd(bool normalize, const float* xyz, const float* gout, float* gxyz, long long n, Scale4 sc, hipStream_t st) {
  const long long blocks = (n + 255) / 256;
  if (normalize)
    hipLaunchKernelGGL((sh_bwd_kernel<LMAX, true>), dim3((unsigned)blocks), dim3(256), 0, st, xyz, gout, gxyz, n, sc);
  else
    hipLaunchKernelGGL((sh_bwd_kernel<LMAX, false>), dim3((unsigned)blocks), dim3(256), 0, st, xyz, gout, gxyz, n, sc);
}

// ---------------------------------------------------------------- generic path
constexpr int kMaxL = 12;
constexpr int kMaxCols = (kMaxL + 1) * (kMaxL + 1);
constexpr int kMaxEntries = 2048;

struct RecEntry {
  unsigned short out_col;  // absolute column of Y^{l+1}_i
  unsigned short in_col;   // absolute column of Y^l_j
  int axis;                // k: 0 x, 1 y, 2 z
  float coef;              // c_l * w3j(l+1, 1, l)[i, k, j]
};

__constant__ RecEntry c_rec[kMaxEntries];
__constant__ int c_rec_end[kMaxL + 1];  // entries for levels < l end at c_rec_end[l]

struct ColMap {
  unsigned char src[kMaxCols];  // output column -> polynomial column
  float scale[kMaxCols];
};

__global__ __launch_bounds__(kWave) void sh_generic_kernel(const float* __restrict__ xyz, float* __restrict__ out,
                                                           long long n, int lmax, int n_out, int normalize,
                                                           const ColMap cmap) {
  extern __shared__ float s_y[];  // [(lmax+1)^2][64]
  const int lane = threadIdx.x;
  for (long long v = (long long)blockIdx.x * kWave + lane; v - lane < n; v += (long long)gridDim.x * kWave) {
    const bool live = v < n;
    float x = 0.f, y = 0.f, z = 0.f;
    if (live) {
      x = xyz[v * 3 + 0];
      y = xyz[v * 3 + 1];
      z = xyz[v * 3 + 2];
    }
    if (normalize) {
      const float inv = 1.0f / fmaxf(sqrtf(x * x + y * y + z * z), 1e-12f);
      x *= inv;
      y *= inv;
      z *= inv;
    }
    s_y[lane] = 1.0f;
    const int n_ent = c_rec_end[lmax];
    int cur = -1;
    float acc = 0.f;
    for (int e = 0; e < n_ent; ++e) {
      const RecEntry r = c_rec[e];
      if ((int)r.out_col != cur) {
        if (cur >= 0) s_y[cur * kWave + lane] = acc;
        cur = r.out_col;
        acc = 0.f;
      }
      const float a = r.axis == 0 ? x : (r.axis == 1 ? y : z);
      acc = fmaf(r.coef * a, s_y[r.in_col * kWave + lane], acc);
    }
    if (cur >= 0) s_y[cur * kWave + lane] = acc;
    if (live) {
      for (int c = 0; c < n_out; ++c) out[v * n_out + c] = cmap.scale[c] * s_y[cmap.src[c] * kWave + lane];
    }
  }
}

// Reverse sweep of the same recurrence for any l list: the forward values of the tile stay in LDS, the adjoint of
// Y^l_j collects coef * a * adj(Y^{l+1}_i) from the level above (entries are ordered by level, so walking them
// backwards finds every adjoint complete), the adjoint of the coordinate a collects coef * Y^l_j * adj(Y^{l+1}_i).
// blockDim.x = 64, or 32 when two tables of 64 columns would not fit in 64 KB of LDS.
__global__ __launch_bounds__(kWave) void sh_generic_bwd_kernel(const float* __restrict__ xyz,
                                                               const float* __restrict__ gout,
                                                               float* __restrict__ gxyz, long long n, int lmax,
                                                               int n_out, int normalize, const ColMap cmap) {
  extern __shared__ float s_mem[];
  const int W = blockDim.x, lane = threadIdx.x;
  const int n_col = (lmax + 1) * (lmax + 1);
  float* s_y = s_mem;
  float* s_g = s_mem + n_col * W;
  for (long long v = (long long)blockIdx.x * W + lane; v - lane < n; v += (long long)gridDim.x * W) {
    const bool live = v < n;
    float x = 0.f, y = 0.f, z = 0.f;
    if (live) {
      x = xyz[v * 3 + 0];
      y = xyz[v * 3 + 1];
      z = xyz[v * 3 + 2];
    }
    const float r = sqrtf(x * x + y * y + z * z);
    const float inv = 1.0f / fmaxf(r, 1e-12f);
    if (normalize) {
      x *= inv;
      y *= inv;
      z *= inv;
    }
    s_y[lane] = 1.0f;
    const int n_ent = c_rec_end[lmax];
    int cur = -1;
    float acc = 0.f;
    for (int e = 0; e < n_ent; ++e) {
      const RecEntry t = c_rec[e];
      if ((int)t.out_col != cur) {
        if (cur >= 0) s_y[cur * W + lane] = acc;
        cur = t.out_col;
        acc = 0.f;
      }
      const float a = t.axis == 0 ? x : (t.axis == 1 ? y : z);
      acc = fmaf(t.coef * a, s_y[t.in_col * W + lane], acc);
    }
    if (cur >= 0) s_y[cur * W + lane] = acc;
    for (int c = 0; c < n_col; ++c) s_g[c * W + lane] = 0.f;
    if (live)
      for (int c = 0; c < n_out; ++c) s_g[cmap.src[c] * W + lane] += cmap.scale[c] * gout[v * n_out + c];
    float gx = 0.f, gy = 0.f, gz = 0.f;
    for (int e = n_ent - 1; e >= 0; --e) {
      const RecEntry t = c_rec[e];
      const float go = s_g[t.out_col * W + lane];
      const float a = t.axis == 0 ? x : (t.axis == 1 ? y : z);
      s_g[t.in_col * W + lane] = fmaf(t.coef * a, go, s_g[t.in_col * W + lane]);
      const float d = t.coef * s_y[t.in_col * W + lane] * go;
      gx += t.axis == 0 ? d : 0.f;
      gy += t.axis == 1 ? d : 0.f;
      gz += t.axis == 2 ? d : 0.f;
    }
    if (normalize) {
      // x / max(|x|, eps): (g - xhat (xhat . g)) / |x| above the clamp, g / eps below it
      const float dot = r > 1e-12f ? x * gx + y * gy + z * gz : 0.f;
      gx = (gx - x * dot) * inv;
      gy = (gy - y * dot) * inv;
      gz = (gz - z * dot) * inv;
    }
    if (live) {
      gxyz[v * 3 + 0] = gx;
      gxyz[v * 3 + 1] = gy;
      gxyz[v * 3 + 2] = gz;
    }
  }
}

std::mutex g_mu;
bool g_tables_ready[64] = {false};

int upload_tables(int dev) {
  if (g_tables_ready[dev]) return E3X_OK;
  std::vector<RecEntry> ent;
  int ends[kMaxL + 1];
  ends[0] = 0;
  // Y^{l+1}_i = c_l sum_{k,j} w3j(l+1,1,l)[i,k,j] x_k Y^l_j ; c_l > 0 from |Y^{l+1}(0,1,0)|^2 = 2l+3
  std::vector<double> pole(1, 1.0);
  for (int l = 0; l < kMaxL; ++l) {
    const auto& C = e3x::wigner_3j(l + 1, 1, l);
    const int d_out = 2 * l + 3, d_in = 2 * l + 1;
    std::vector<double> raw(d_out, 0.0);
    double nrm = 0;
    for (int i = 0; i < d_out; ++i) {
      for (int j = 0; j < d_in; ++j) raw[i] += C[(i * 3 + 1) * d_in + j] * pole[j];
      nrm += raw[i] * raw[i];
    }
    const double cl = std::sqrt((2.0 * l + 3.0) / nrm);
    for (auto& v : raw) v *= cl;
    pole = raw;
    for (int i = 0; i < d_out; ++i)
      for (int k = 0; k < 3; ++k)
        for (int j = 0; j < d_in; ++j) {
          const double c = C[(i * 3 + k) * d_in + j];
          if (c != 0.0) {
            RecEntry r;
            r.out_col = (unsigned short)((l + 1) * (l + 1) + i);
            r.in_col = (unsigned short)(l * l + j);
            r.axis = k;
            r.coef = (float)(cl * c);
            ent.push_back(r);
          }
        }
    ends[l + 1] = (int)ent.size();
  }
  if ((int)ent.size() > kMaxEntries) return e3x::fail(E3X_ERR_INVALID, "sh: recurrence table overflow");
  if (hipMemcpyToSymbol(HIP_SYMBOL(c_rec), ent.data(), ent.size() * sizeof(RecEntry)) != hipSuccess ||
      hipMemcpyToSymbol(HIP_SYMBOL(c_rec_end), ends, sizeof(ends)) != hipSuccess)
    return e3x::fail(E3X_ERR_HIP, "sh: uploading the recurrence table failed");
  g_tables_ready[dev] = true;
  return E3X_OK;
}

template <int LMAX>
void launch_tile(bool normalize, const float* xyz, float* out, long long n, Scale4 sc, hipStream_t st) {
  const long long tiles = (n + kWave - 1) / kWave;
  long long blocks = (tiles + kWavesPerBlock - 1) / kWavesPerBlock;
  // one tile per wavefront: on this chip a grid that covers the data once streams faster than a
  // capped grid with a grid-stride loop (the loop in the kernel only runs for n > 2^31 * 256 vectors)
  if (blocks > 0x7fffffffLL) blocks = 0x7fffffffLL;
  if (normalize)
    hipLaunchKernelGGL((sh_tile_kernel<LMAX, true>), dim3((unsigned)blocks), dim3(kWave * kWavesPerBlock), 0, st, xyz,
                       out, n, sc);
  else
    hipLaunchKernelGGL((sh_tile_kernel<LMAX, false>), dim3((unsigned)blocks), dim3(kWave * kWavesPerBlock), 0, st,
                       xyz, out, n, sc);
}

}  // namespace

extern "C" int e3x_sh_forward(const int32_t* ls, int32_t n_ls, int32_t normalize, int32_t normalization,
                              const void* xyz, void* out, int64_t n, int32_t dtype, void* stream) {
  if (!ls || n_ls <= 0 || n < 0) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_forward: empty l list or negative n");
  if (dtype != E3X_F32) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_forward: only fp32 storage is implemented");
  if (normalization < 0 || normalization > 2)
    return e3x::fail(E3X_ERR_INVALID, "e3x_sh_forward: normalization must be integral, component or norm");
  int lmax = 0, n_out = 0;
  bool is_range = true;
  for (int i = 0; i < n_ls; ++i) {
    if (ls[i] < 0 || ls[i] > kMaxL)
      return e3x::fail(E3X_ERR_INVALID, "spherical_harmonics maximum l implemented is 12");
    lmax = ls[i] > lmax ? ls[i] : lmax;
    is_range = is_range && ls[i] == i;
    n_out += 2 * ls[i] + 1;
  }
  if (n_out > kMaxCols) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_forward: more than 169 output columns");
  if (n == 0) return E3X_OK;
  if (!xyz || !out) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_forward: null pointer");
  hipStream_t st = (hipStream_t)stream;
  auto lscale = [&](int l) -> float {
    if (normalization == E3X_NORM_INTEGRAL) return (float)(1.0 / std::sqrt(4.0 * M_PI));
    if (normalization == E3X_NORM_NORM) return (float)(1.0 / std::sqrt(2.0 * l + 1.0));
    return 1.0f;
  };
  const bool aligned = ((uintptr_t)xyz % 16 == 0) && ((uintptr_t)out % 16 == 0);
  if (is_range && lmax <= 3 && aligned) {
    Scale4 sc;
    for (int l = 0; l < 4; ++l) sc.s[l] = lscale(l);
    const float* px = (const float*)xyz;
    float* po = (float*)out;
    switch (lmax) {
      case 0: launch_tile<0>(normalize, px, po, n, sc, st); break;
      case 1: launch_tile<1>(normalize, px, po, n, sc, st); break;
      case 2: launch_tile<2>(normalize, px, po, n, sc, st); break;
      default: launch_tile<3>(normalize, px, po, n, sc, st); break;
    }
  } else {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return e3x::fail(E3X_ERR_HIP, "hipGetDevice failed");
    std::lock_guard<std::mutex> lock(g_mu);
    int rc = upload_tables(dev);
    if (rc) return rc;
    ColMap cm;
    int c = 0;
    for (int i = 0; i < n_ls; ++i)
      for (int m = 0; m < 2 * ls[i] + 1; ++m, ++c) {
        cm.src[c] = (unsigned char)(ls[i] * ls[i] + m);
        cm.scale[c] = lscale(ls[i]);
      }
    long long blocks = (n + kWave - 1) / kWave;
    if (blocks > 256 * 16) blocks = 256 * 16;
    const size_t shmem = (size_t)(lmax + 1) * (lmax + 1) * kWave * sizeof(float);
    hipLaunchKernelGGL(sh_generic_kernel, dim3((unsigned)blocks), dim3(kWave), shmem, st, (const float*)xyz,
                       (float*)out, (long long)n, lmax, n_out, (int)normalize, cm);
  }
  if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_sh_forward: kernel launch failed");
  return E3X_OK;
}

extern "C" int e3x_sh_backward(const int32_t* ls, int32_t n_ls, int32_t normalize, int32_t normalization,
                               const void* xyz, const void* grad_out, void* grad_xyz, int64_t n, int32_t dtype,
                               void* stream) {
  if (!ls || n_ls <= 0 || n < 0) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward: empty l list or negative n");
  if (dtype != E3X_F32) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward: only fp32 storage is implemented");
  if (normalization < 0 || normalization > 2)
    return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward: normalization must be integral, component or norm");
  int lmax = 0, n_out = 0;
  bool is_range = true;
  for (int i = 0; i < n_ls; ++i) {
    if (ls[i] < 0 || ls[i] > kMaxL) return e3x::fail(E3X_ERR_INVALID, "spherical_harmonics maximum l implemented is 12");
    lmax = ls[i] > lmax ? ls[i] : lmax;
    is_range = is_range && ls[i] == i;
    n_out += 2 * ls[i] + 1;
  }
  if (n_out > kMaxCols) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward: more than 169 output columns");
  if (n == 0) return E3X_OK;
  if (!xyz || !grad_out || !grad_xyz) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward: null pointer");
  if (n >= (1LL << 31) * 256) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward: too many vectors for one launch");
  hipStream_t st = (hipStream_t)stream;
  if (!is_range || lmax > 3) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return e3x::fail(E3X_ERR_HIP, "hipGetDevice failed");
    std::lock_guard<std::mutex> lock(g_mu);
    int rc = upload_tables(dev);
    if (rc) return rc;
    ColMap cm;
    int c = 0;
    for (int i = 0; i < n_ls; ++i)
      for (int m = 0; m < 2 * ls[i] + 1; ++m, ++c) {
        cm.src[c] = (unsigned char)(ls[i] * ls[i] + m);
        cm.scale[c] = normalization == E3X_NORM_INTEGRAL ? (float)(1.0 / std::sqrt(4.0 * M_PI))
                      : normalization == E3X_NORM_NORM   ? (float)(1.0 / std::sqrt(2.0 * ls[i] + 1.0))
                                                         : 1.0f;
      }
    const int n_col = (lmax + 1) * (lmax + 1);
    const int width = 2 * n_col * kWave * (int)sizeof(float) <= 65536 ? kWave : kWave / 2;
    long long blocks = (n + width - 1) / width;
    if (blocks > 256 * 16) blocks = 256 * 16;
    const size_t shmem = (size_t)2 * n_col * width * sizeof(float);
    hipLaunchKernelGGL(sh_generic_bwd_kernel, dim3((unsigned)blocks), dim3(width), shmem, st, (const float*)xyz,
                       (const float*)grad_out, (float*)grad_xyz, (long long)n, lmax, n_out, (int)normalize, cm);
    if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_sh_backward: kernel launch failed");
    return E3X_OK;
  }
  Scale4 sc;
  for (int l = 0; l < 4; ++l) {
    sc.s[l] = 1.0f;
    if (normalization == E3X_NORM_INTEGRAL) sc.s[l] = (float)(1.0 / std::sqrt(4.0 * M_PI));
    if (normalization == E3X_NORM_NORM) sc.s[l] = (float)(1.0 / std::sqrt(2.0 * l + 1.0));
  }
  const float *px = (const float*)xyz, *pg = (const float*)grad_out;
  float* po = (float*)grad_xyz;
  switch (lmax) {
    case 0: launch_bwd<0>(normalize, px, pg, po, n, sc, st); break;
    case 1: launch_bwd<1>(normalize, px, pg, po, n, sc, st); break;
    case 2: launch_bwd<2>(normalize, px, pg, po, n, sc, st); break;
    default: launch_bwd<3>(normalize, px, pg, po, n, sc, st); break;
  }
  if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_sh_backward: kernel launch failed");
  return E3X_OK;
}

extern "C" int e3x_sh_backward2(const int32_t* ls, int32_t n_ls, int32_t normalize, int32_t normalization,
                                const void* xyz, const void* grad_out, const void* cot_xyz, void* grad_grad_out,
                                void* grad_xyz, int64_t n, int32_t dtype, void* stream) {
  if (!ls || n_ls <= 0 || n < 0) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward2: empty l list or negative n");
  if (dtype != E3X_F32) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward2: only fp32 storage is implemented");
  if (normalization < 0 || normalization > 2)
    return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward2: normalization must be integral, component or norm");
  for (int i = 0; i < n_ls; ++i)
    if (ls[i] != i || i > 3)
      return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward2: second derivatives are implemented for the l lists 0 .. lmax <= 3");
  if (n == 0) return E3X_OK;
  if (!xyz || !grad_out || !cot_xyz || !grad_grad_out || !grad_xyz) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward2: null pointer");
  if (n >= (1LL << 31) * 256) return e3x::fail(E3X_ERR_INVALID, "e3x_sh_backward2: too many vectors for one launch");
  hipStream_t st = (hipStream_t)stream;
  Scale4 sc;
  for (int l = 0; l < 4; ++l) {
    sc.s[l] = 1.0f;
    if (normalization == E3X_NORM_INTEGRAL) sc.s[l] = (float)(1.0 / std::sqrt(4.0 * M_PI));
    if (normalization == E3X_NORM_NORM) sc.s[l] = (float)(1.0 / std::sqrt(2.0 * l + 1.0));
  }
  const float *px = (const float*)xyz, *pg = (const float*)grad_out, *pc = (const float*)cot_xyz;
  float *pgg = (float*)grad_grad_out, *po = (float*)grad_xyz;
  switch (n_ls - 1) {
    case 0: launch_bwd2<0>(normalize, px, pg, pc, pgg, po, n, sc, st); break;
    case 1: launch_bwd2<1>(normalize, px, pg, pc, pgg, po, n, sc, st); break;
    case 2: launch_bwd2<2>(normalize, px, pg, pc, pgg, po, n, sc, st); break;
    default: launch_bwd2<3>(normalize, px, pg, pc, pgg, po, n, sc, st); break;
  }
  if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_sh_backward2: kernel launch failed");
  return E3X_OK;
}
