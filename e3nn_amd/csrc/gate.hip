// Gated non-linearity of equivariant features (gfx950): scalars go through normalised activation functions, every
// copy of a non-scalar irrep is multiplied by its own activated gate scalar.  Replaces nn.Gate.forward
// (e3nn/nn/_gate.py:121-144: Extract -> Activation -> ElementwiseTensorProduct -> cat, about a dozen ATen kernels and
// three intermediates) and, with no gated part, nn.Activation.forward (e3nn/nn/_activation.py:78-104).  One pass over
// the row: HBM-bound, (in_dim + out_dim) * 4 bytes per row (2 bytes per element in bf16 storage; fp32 arithmetic).
#include <hip/hip_runtime.h>

#include <cstdint>

#include "e3x_internal.h"

namespace {

constexpr int kMaxBlocks = 16;

struct Tables {
  e3x_act_block act[kMaxBlocks];
  e3x_gate_block gate[kMaxBlocks];
  int n_act, n_gate;
};

// rows are stored as fp32 or bf16; the arithmetic is fp32 either way
__device__ __forceinline__ float ld(const float* p, long long i) { return p[i]; }
__device__ __forceinline__ float ld(const __bf16* p, long long i) { return (float)p[i]; }
__device__ __forceinline__ void st(float* p, long long i, float v) { p[i] = v; }
__device__ __forceinline__ void st(__bf16* p, long long i, float v) { p[i] = (__bf16)v; }

__device__ __forceinline__ float sigmoidf(float x) { return 1.f / (1.f + __expf(-x)); }

// value and derivative of activation `kind` at x
__device__ __forceinline__ void activation(int kind, float x, float& f, float& df) {
  switch (kind) {
    case E3X_ACT_SILU: {
      const float s = sigmoidf(x);
      f = x * s;
      df = s * (1.f + x * (1.f - s));
      break;
    }
    case E3X_ACT_TANH: {
      f = tanhf(x);
      df = 1.f - f * f;
      break;
    }
    case E3X_ACT_SIGMOID: {
      f = sigmoidf(x);
      df = f * (1.f - f);
      break;
    }
    case E3X_ACT_ABS: {
      f = fabsf(x);
      df = x > 0.f ? 1.f : (x < 0.f ? -1.f : 0.f);
      break;
    }
    case E3X_ACT_RELU: {
      f = x > 0.f ? x : 0.f;
      df = x > 0.f ? 1.f : 0.f;
      break;
    }
    default: {
      f = x;
      df = 1.f;
    }
  }
}

// second derivative of activation `kind` at x (0 for the piecewise linear ones, away from their kink)
__device__ __forceinline__ float activation_d2(int kind, float x) {
  switch (kind) {
    case E3X_ACT_SILU: {
      const float s = sigmoidf(x);
      return s * (1.f - s) * (2.f + x * (1.f - 2.f * s));
    }
    case E3X_ACT_TANH: {
      const float f = tanhf(x);
      return -2.f * f * (1.f - f * f);
    }
    case E3X_ACT_SIGMOID: {
      const float f = sigmoidf(x);
      return f * (1.f - f) * (1.f - 2.f * f);
    }
    default: return 0.f;
  }
}

// Thread (tx, ty) of a 64 x 4 block owns column 64 blockIdx.x + tx and walks rows 4 blockIdx.y + ty, + 4 gridDim.y, ...:
// the block tables are searched once per thread, consecutive lanes touch consecutive columns of a row.
constexpr int kCols = 64, kRows = 4;

template <class T>
__global__ __launch_bounds__(kCols* kRows) void gate_fwd_kernel(Tables t, const T* __restrict__ x,
                                                                T* __restrict__ out, long long n_rows, int in_dim,
                                                                int out_dim) {
  const int c = blockIdx.x * kCols + (threadIdx.x % kCols);
  if (c >= out_dim) return;
  int kind = -1, src = 0, gate = -1;  // kind < 0: no block covers this column
  float cst = 0.f;
  for (int b = 0; b < t.n_act; ++b) {
    const e3x_act_block& a = t.act[b];
    if (c >= a.offset_out && c < a.offset_out + a.count) kind = a.act, cst = a.cst, src = a.offset_in + (c - a.offset_out);
  }
  for (int b = 0; b < t.n_gate; ++b) {
    const e3x_gate_block& g = t.gate[b];
    if (c >= g.offset_out && c < g.offset_out + g.mul * g.dim) {
      const int rel = c - g.offset_out;
      kind = g.act, cst = g.cst, src = g.gated_offset_in + rel, gate = g.gate_offset_in + rel / g.dim;
    }
  }
  for (long long z = (long long)blockIdx.y * kRows + threadIdx.x / kCols; z < n_rows; z += (long long)gridDim.y * kRows) {
    const T* row = x + z * in_dim;
    float v = 0.f;
    if (kind >= 0) {
      float f, df;
      activation(kind, ld(row, gate >= 0 ? gate : src), f, df);
      v = gate >= 0 ? cst * f * ld(row, src) : cst * f;
    }
    st(out, z * out_dim + c, v);
  }
}

// the same walk over the input columns: a scalar or gated component takes one term, a gate sums over its irrep
template <class T>
__global__ __launch_bounds__(kCols* kRows) void gate_bwd_kernel(Tables t, const T* __restrict__ x,
                                                                const T* __restrict__ gout, T* __restrict__ gx,
                                                                long long n_rows, int in_dim, int out_dim) {
  const int c = blockIdx.x * kCols + (threadIdx.x % kCols);
  if (c >= in_dim) return;
  // roles of this input column (a column can play at most one role per block kind)
  int a_kind = -1, a_out = 0;
  float a_cst = 0.f;
  int y_kind = -1, y_out = 0, y_gate = 0;  // gated component
  float y_cst = 0.f;
  int g_kind = -1, g_out = 0, g_src = 0, g_dim = 0;  // gate scalar
  float g_cst = 0.f;
  for (int b = 0; b < t.n_act; ++b) {
    const e3x_act_block& a = t.act[b];
    if (c >= a.offset_in && c < a.offset_in + a.count) a_kind = a.act, a_cst = a.cst, a_out = a.offset_out + (c - a.offset_in);
  }
  for (int b = 0; b < t.n_gate; ++b) {
    const e3x_gate_block& g = t.gate[b];
    if (c >= g.gated_offset_in && c < g.gated_offset_in + g.mul * g.dim) {
      const int rel = c - g.gated_offset_in;
      y_kind = g.act, y_cst = g.cst, y_out = g.offset_out + rel, y_gate = g.gate_offset_in + rel / g.dim;
    }
    if (c >= g.gate_offset_in && c < g.gate_offset_in + g.mul) {
      const int u = c - g.gate_offset_in;
      g_kind = g.act, g_cst = g.cst, g_out = g.offset_out + u * g.dim, g_src = g.gated_offset_in + u * g.dim, g_dim = g.dim;
    }
  }
  for (long long z = (long long)blockIdx.y * kRows + threadIdx.x / kCols; z < n_rows; z += (long long)gridDim.y * kRows) {
    const T* row = x + z * in_dim;
    const T* grow = gout + z * out_dim;
    float v = 0.f, f, df;
    if (a_kind >= 0) {
      activation(a_kind, ld(row, c), f, df);
      v += a_cst * df * ld(grow, a_out);
    }
    if (y_kind >= 0) {
      activation(y_kind, ld(row, y_gate), f, df);
      v += y_cst * f * ld(grow, y_out);
    }
    if (g_kind >= 0) {
      activation(g_kind, ld(row, c), f, df);
      float s = 0.f;
      for (int m = 0; m < g_dim; ++m) s += ld(grow, g_out + m) * ld(row, g_src + m);
      v += g_cst * df * s;
    }
    st(gx, z * in_dim + c, v);
  }
}

// The derivative of the backward pass, for a cotangent `cot` on its result gx: with Phi = <cot, gx(x, gout)>,
//   gg = dPhi/dgout (walk over the output columns) and gx2 = dPhi/dx (walk over the input columns).
// A scalar block contributes cot * cst * a'(x) to gg and cot * gout * cst * a''(x) to gx2; a gated component with gate
// s, value y, output gradient g and cotangents (cs, cy): gg = cy cst a(s) + cs cst a'(s) y,
// dPhi/dy = cs cst a'(s) g, dPhi/ds = cst a'(s) sum(cy g) + cs cst a''(s) sum(g y).
template <class T>
__global__ __launch_bounds__(kCols* kRows) void gate_bwd2_gg_kernel(Tables t, const T* __restrict__ x,
                                                                    const T* __restrict__ cot, T* __restrict__ gg,
                                                                    long long n_rows, int in_dim, int out_dim) {
  const int c = blockIdx.x * kCols + (threadIdx.x % kCols);
  if (c >= out_dim) return;
  int kind = -1, src = 0, gate = -1;
  float cst = 0.f;
  for (int b = 0; b < t.n_act; ++b) {
    const e3x_act_block& a = t.act[b];
    if (c >= a.offset_out && c < a.offset_out + a.count) kind = a.act, cst = a.cst, src = a.offset_in + (c - a.offset_out);
  }
  for (int b = 0; b < t.n_gate; ++b) {
    const e3x_gate_block& g = t.gate[b];
    if (c >= g.offset_out && c < g.offset_out + g.mul * g.dim) {
      const int rel = c - g.offset_out;
      kind = g.act, cst = g.cst, src = g.gated_offset_in + rel, gate = g.gate_offset_in + rel / g.dim;
    }
  }
  for (long long z = (long long)blockIdx.y * kRows + threadIdx.x / kCols; z < n_rows; z += (long long)gridDim.y * kRows) {
    const T* row = x + z * in_dim;
    const T* crow = cot + z * in_dim;
    float v = 0.f;
    if (kind >= 0) {
      float f, df;
      activation(kind, ld(row, gate >= 0 ? gate : src), f, df);
      v = gate >= 0 ? cst * (ld(crow, src) * f + ld(crow, gate) * df * ld(row, src)) : cst * df * ld(crow, src);
    }
    st(gg, z * out_dim + c, v);
  }
}

template <class T>
__global__ __launch_bounds__(kCols* kRows) void gate_bwd2_gx_kernel(Tables t, const T* __restrict__ x,
                                                                    const T* __restrict__ gout,
                                                                    const T* __restrict__ cot, T* __restrict__ gx2,
                                                                    long long n_rows, int in_dim, int out_dim) {
  const int c = blockIdx.x * kCols + (threadIdx.x % kCols);
  if (c >= in_dim) return;
  int a_kind = -1, a_out = 0;
  float a_cst = 0.f;
  int y_kind = -1, y_out = 0, y_gate = 0;
  float y_cst = 0.f;
  int g_kind = -1, g_out = 0, g_src = 0, g_dim = 0;
  float g_cst = 0.f;
  for (int b = 0; b < t.n_act; ++b) {
    const e3x_act_block& a = t.act[b];
    if (c >= a.offset_in && c < a.offset_in + a.count) a_kind = a.act, a_cst = a.cst, a_out = a.offset_out + (c - a.offset_in);
  }
  for (int b = 0; b < t.n_gate; ++b) {
    const e3x_gate_block& g = t.gate[b];
    if (c >= g.gated_offset_in && c < g.gated_offset_in + g.mul * g.dim) {
      const int rel = c - g.gated_offset_in;
      y_kind = g.act, y_cst = g.cst, y_out = g.offset_out + rel, y_gate = g.gate_offset_in + rel / g.dim;
    }
    if (c >= g.gate_offset_in && c < g.gate_offset_in + g.mul) {
      const int u = c - g.gate_offset_in;
      g_kind = g.act, g_cst = g.cst, g_out = g.offset_out + u * g.dim, g_src = g.gated_offset_in + u * g.dim, g_dim = g.dim;
    }
  }
  for (long long z = (long long)blockIdx.y * kRows + threadIdx.x / kCols; z < n_rows; z += (long long)gridDim.y * kRows) {
    const T* row = x + z * in_dim;
    const T* grow = gout + z * out_dim;
    const T* crow = cot + z * in_dim;
    float v = 0.f, f, df;
    if (a_kind >= 0) v += a_cst * activation_d2(a_kind, ld(row, c)) * ld(grow, a_out) * ld(crow, c);
    if (y_kind >= 0) {
      activation(y_kind, ld(row, y_gate), f, df);
      v += y_cst * df * ld(grow, y_out) * ld(crow, y_gate);
    }
    if (g_kind >= 0) {
      activation(g_kind, ld(row, c), f, df);
      float s_cg = 0.f, s_gy = 0.f;
      for (int m = 0; m < g_dim; ++m) {
        s_cg += ld(crow, g_src + m) * ld(grow, g_out + m);
        s_gy += ld(grow, g_out + m) * ld(row, g_src + m);
      }
      v += g_cst * (df * s_cg + activation_d2(g_kind, ld(row, c)) * ld(crow, c) * s_gy);
    }
    st(gx2, z * in_dim + c, v);
  }
}

// One activation over whole contiguous rows (an Activation on n x0e, the hidden layer of a radial network): the
// tensor is one flat array, 16 bytes per thread and access.
__global__ __launch_bounds__(256) void act_flat_fwd_kernel(int kind, float cst, const float4* __restrict__ x,
                                                           float4* __restrict__ out, long long n4) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n4; i += (long long)gridDim.x * 256) {
    const float4 v = x[i];
    float f[4], df;
    activation(kind, v.x, f[0], df);
    activation(kind, v.y, f[1], df);
    activation(kind, v.z, f[2], df);
    activation(kind, v.w, f[3], df);
    out[i] = make_float4(cst * f[0], cst * f[1], cst * f[2], cst * f[3]);
  }
}

__global__ __launch_bounds__(256) void act_flat_bwd_kernel(int kind, float cst, const float4* __restrict__ x,
                                                           const float4* __restrict__ gout, float4* __restrict__ gx,
                                                           long long n4) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n4; i += (long long)gridDim.x * 256) {
    const float4 v = x[i], g = gout[i];
    float f, d[4];
    activation(kind, v.x, f, d[0]);
    activation(kind, v.y, f, d[1]);
    activation(kind, v.z, f, d[2]);
    activation(kind, v.w, f, d[3]);
    gx[i] = make_float4(cst * d[0] * g.x, cst * d[1] * g.y, cst * d[2] * g.z, cst * d[3] * g.w);
  }
}

// true when the tables describe one activation applied to every column of contiguous, 16-byte aligned rows
bool is_flat(const Tables& t, int64_t Z, int64_t in_dim, int64_t out_dim, const void* a, const void* b, const void* c) {
  if (t.n_gate != 0 || t.n_act != 1 || in_dim != out_dim) return false;
  const e3x_act_block& k = t.act[0];
  if (k.offset_in != 0 || k.offset_out != 0 || k.count != in_dim) return false;
  if ((Z * in_dim) % 4) return false;
  return ((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0) && (!c || (uintptr_t)c % 16 == 0);
}

unsigned flat_grid(long long n4) {
  long long b = (n4 + 255) / 256;
  if (b > 256 * 32) b = 256 * 32;
  return (unsigned)(b < 1 ? 1 : b);
}

// grid of the column-walk kernels: all column blocks, enough row blocks for a few workgroups per CU
dim3 walk_grid(int64_t Z, int64_t dim) {
  const long long cb = (dim + kCols - 1) / kCols;
  long long rb = (Z + kRows - 1) / kRows;
  const long long want = (256LL * 16 + cb - 1) / cb;
  if (rb > want) rb = want;
  if (rb > 65535) rb = 65535;
  return dim3((unsigned)cb, (unsigned)rb);
}

int fill_tables(const char* who, const e3x_act_block* acts, int n_acts, const e3x_gate_block* gates, int n_gates,
                int64_t in_dim, int64_t out_dim, Tables* t) {
  if (n_acts < 0 || n_gates < 0 || n_acts > kMaxBlocks || n_gates > kMaxBlocks)
    return e3x::fail(E3X_ERR_INVALID, std::string(who) + ": at most 16 scalar blocks and 16 gated blocks");
  if ((n_acts && !acts) || (n_gates && !gates)) return e3x::fail(E3X_ERR_INVALID, std::string(who) + ": null block table");
  if (in_dim < 0 || out_dim < 0 || in_dim >= (1 << 30) || out_dim >= (1 << 30))
    return e3x::fail(E3X_ERR_INVALID, std::string(who) + ": bad row length");
  t->n_act = n_acts;
  t->n_gate = n_gates;
  for (int i = 0; i < n_acts; ++i) {
    const e3x_act_block& a = acts[i];
    if (a.count < 0 || a.offset_in < 0 || a.offset_out < 0 || a.offset_in + (int64_t)a.count > in_dim ||
        a.offset_out + (int64_t)a.count > out_dim || a.act < 0 || a.act > E3X_ACT_RELU)
      return e3x::fail(E3X_ERR_INVALID, std::string(who) + ": scalar block outside the rows or unknown activation");
    t->act[i] = a;
  }
  for (int i = 0; i < n_gates; ++i) {
    const e3x_gate_block& g = gates[i];
    const int64_t n = (int64_t)g.mul * g.dim;
    if (g.mul < 0 || g.dim < 1 || g.gate_offset_in < 0 || g.gated_offset_in < 0 || g.offset_out < 0 ||
        g.gate_offset_in + (int64_t)g.mul > in_dim || g.gated_offset_in + n > in_dim || g.offset_out + n > out_dim ||
        g.act < 0 || g.act > E3X_ACT_RELU)
      return e3x::fail(E3X_ERR_INVALID, std::string(who) + ": gated block outside the rows or unknown activation");
    t->gate[i] = g;
  }
  return E3X_OK;
}

}  // namespace

extern "C" int e3x_gate_forward(const e3x_act_block* acts, int32_t n_acts, const e3x_gate_block* gates, int32_t n_gates,
                                const void* x, void* out, int64_t Z, int64_t in_dim, int64_t out_dim, int32_t dtype,
                                void* stream) {
  if (dtype != E3X_F32 && dtype != E3X_BF16) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_forward: storage is fp32 or bf16");
  Tables t;
  int rc = fill_tables("e3x_gate_forward", acts, n_acts, gates, n_gates, in_dim, out_dim, &t);
  if (rc) return rc;
  if (Z < 0) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_forward: negative batch");
  if (Z == 0 || out_dim == 0) return E3X_OK;
  if (!x || !out) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_forward: null pointer");
  if (dtype == E3X_F32 && is_flat(t, Z, in_dim, out_dim, x, out, nullptr)) {
    const long long n4 = Z * in_dim / 4;
    hipLaunchKernelGGL(act_flat_fwd_kernel, dim3(flat_grid(n4)), dim3(256), 0, (hipStream_t)stream, t.act[0].act, t.act[0].cst,
                       (const float4*)x, (float4*)out, n4);
    if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_gate_forward: kernel launch failed");
    return E3X_OK;
  }
  if (dtype == E3X_BF16)
    hipLaunchKernelGGL(gate_fwd_kernel<__bf16>, walk_grid(Z, out_dim), dim3(kCols * kRows), 0, (hipStream_t)stream, t,
                       (const __bf16*)x, (__bf16*)out, (long long)Z, (int)in_dim, (int)out_dim);
  else
    hipLaunchKernelGGL(gate_fwd_kernel<float>, walk_grid(Z, out_dim), dim3(kCols * kRows), 0, (hipStream_t)stream, t,
                       (const float*)x, (float*)out, (long long)Z, (int)in_dim, (int)out_dim);
  if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_gate_forward: kernel launch failed");
  return E3X_OK;
}

extern "C" int e3x_gate_backward(const e3x_act_block* acts, int32_t n_acts, const e3x_gate_block* gates, int32_t n_gates,
                                 const void* x, const void* grad_out, void* grad_x, int64_t Z, int64_t in_dim,
                                 int64_t out_dim, int32_t dtype, void* stream) {
  if (dtype != E3X_F32 && dtype != E3X_BF16) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward: storage is fp32 or bf16");
  Tables t;
  int rc = fill_tables("e3x_gate_backward", acts, n_acts, gates, n_gates, in_dim, out_dim, &t);
  if (rc) return rc;
  if (Z < 0) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward: negative batch");
  if (Z == 0 || in_dim == 0) return E3X_OK;
  if (!x || !grad_out || !grad_x) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward: null pointer");
  if (dtype == E3X_F32 && is_flat(t, Z, in_dim, out_dim, x, grad_out, grad_x)) {
    const long long n4 = Z * in_dim / 4;
    hipLaunchKernelGGL(act_flat_bwd_kernel, dim3(flat_grid(n4)), dim3(256), 0, (hipStream_t)stream, t.act[0].act, t.act[0].cst,
                       (const float4*)x, (const float4*)grad_out, (float4*)grad_x, n4);
    if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_gate_backward: kernel launch failed");
    return E3X_OK;
  }
  if (dtype == E3X_BF16)
    hipLaunchKernelGGL(gate_bwd_kernel<__bf16>, walk_grid(Z, in_dim), dim3(kCols * kRows), 0, (hipStream_t)stream, t,
                       (const __bf16*)x, (const __bf16*)grad_out, (__bf16*)grad_x, (long long)Z, (int)in_dim, (int)out_dim);
  else
    hipLaunchKernelGGL(gate_bwd_kernel<float>, walk_grid(Z, in_dim), dim3(kCols * kRows), 0, (hipStream_t)stream, t,
                       (const float*)x, (const float*)grad_out, (float*)grad_x, (long long)Z, (int)in_dim, (int)out_dim);
  if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_gate_backward: kernel launch failed");
  return E3X_OK;
}

extern "C" int e3x_gate_backward2(const e3x_act_block* acts, int32_t n_acts, const e3x_gate_block* gates, int32_t n_gates,
                                  const void* x, const void* grad_out, const void* cot_x, void* grad_grad_out, void* grad_x,
                                  int64_t Z, int64_t in_dim, int64_t out_dim, int32_t dtype, void* stream) {
  if (dtype != E3X_F32 && dtype != E3X_BF16) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward2: storage is fp32 or bf16");
  Tables t;
  int rc = fill_tables("e3x_gate_backward2", acts, n_acts, gates, n_gates, in_dim, out_dim, &t);
  if (rc) return rc;
  if (Z < 0) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward2: negative batch");
  if (Z == 0) return E3X_OK;
  if ((in_dim && (!x || !cot_x || !grad_x)) || (out_dim && (!grad_out || !grad_grad_out)))
    return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward2: null pointer");
  if (out_dim) {
    if (dtype == E3X_BF16)
      hipLaunchKernelGGL(gate_bwd2_gg_kernel<__bf16>, walk_grid(Z, out_dim), dim3(kCols * kRows), 0, (hipStream_t)stream, t,
                         (const __bf16*)x, (const __bf16*)cot_x, (__bf16*)grad_grad_out, (long long)Z, (int)in_dim, (int)out_dim);
    else
      hipLaunchKernelGGL(gate_bwd2_gg_kernel<float>, walk_grid(Z, out_dim), dim3(kCols * kRows), 0, (hipStream_t)stream, t,
                         (const float*)x, (const float*)cot_x, (float*)grad_grad_out, (long long)Z, (int)in_dim, (int)out_dim);
    if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_gate_backward2: kernel launch failed");
  }
  if (in_dim) {
    if (dtype == E3X_BF16)
      hipLaunchKernelGGL(gate_bwd2_gx_kernel<__bf16>, walk_grid(Z, in_dim), dim3(kCols * kRows), 0, (hipStream_t)stream, t,
                         (const __bf16*)x, (const __bf16*)grad_out, (const __bf16*)cot_x, (__bf16*)grad_x, (long long)Z, (int)in_dim,
                         (int)out_dim);
    else
      hipLaunchKernelGGL(gate_bwd2_gx_kernel<float>, walk_grid(Z, in_dim), dim3(kCols * kRows), 0, (hipStream_t)stream, t,
                         (const float*)x, (const float*)grad_out, (const float*)cot_x, (float*)grad_x, (long long)Z, (int)in_dim,
                         (int)out_dim);
    if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_gate_backward2: kernel launch failed");
  }
  return E3X_OK;
}
