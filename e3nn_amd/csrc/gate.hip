// Gated non-linearity of equivariant features (gfx950): scalars go through normalised activation functions, every
// copy of a non-scalar irrep is multiplied by its own activated gate scalar.  Replaces nn.Gate.forward
// (e3nn/nn/_gate.py:121-144: Extract -> Activation -> ElementwiseTensorProduct -> cat, about a dozen ATen kernels and
// three intermediates) and, with no gated part, nn.Activation.forward (e3nn/nn/_activation.py:78-104).  One pass over
// the row: HBM-bound, (in_dim + out_dim) * 4 bytes per row.
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

// one thread per output element (row z, column c): consecutive threads write consecutive columns
__global__ __launch_bounds__(256) void gate_fwd_kernel(Tables t, const float* __restrict__ x, float* __restrict__ out,
                                                       long long n_rows, int in_dim, int out_dim) {
  const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
  if (id >= n_rows * out_dim) return;
  const long long z = id / out_dim;
  const int c = (int)(id - z * out_dim);
  const float* row = x + z * in_dim;
  float v = 0.f;
  for (int b = 0; b < t.n_act; ++b) {
    const e3x_act_block& a = t.act[b];
    if (c >= a.offset_out && c < a.offset_out + a.count) {
      float f, df;
      activation(a.act, row[a.offset_in + (c - a.offset_out)], f, df);
      v = a.cst * f;
    }
  }
  for (int b = 0; b < t.n_gate; ++b) {
    const e3x_gate_block& g = t.gate[b];
    if (c >= g.offset_out && c < g.offset_out + g.mul * g.dim) {
      const int rel = c - g.offset_out, u = rel / g.dim;
      float f, df;
      activation(g.act, row[g.gate_offset_in + u], f, df);
      v = g.cst * f * row[g.gated_offset_in + rel];
    }
  }
  out[id] = v;
}

// one thread per input element: scalars and gated components take one term, a gate sums over its irrep's components
__global__ __launch_bounds__(256) void gate_bwd_kernel(Tables t, const float* __restrict__ x,
                                                       const float* __restrict__ gout, float* __restrict__ gx,
                                                       long long n_rows, int in_dim, int out_dim) {
  const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
  if (id >= n_rows * in_dim) return;
  const long long z = id / in_dim;
  const int c = (int)(id - z * in_dim);
  const float* row = x + z * in_dim;
  const float* grow = gout + z * out_dim;
  float v = 0.f;
  for (int b = 0; b < t.n_act; ++b) {
    const e3x_act_block& a = t.act[b];
    if (c >= a.offset_in && c < a.offset_in + a.count) {
      float f, df;
      activation(a.act, row[c], f, df);
      v += a.cst * df * grow[a.offset_out + (c - a.offset_in)];
    }
  }
  for (int b = 0; b < t.n_gate; ++b) {
    const e3x_gate_block& g = t.gate[b];
    if (c >= g.gated_offset_in && c < g.gated_offset_in + g.mul * g.dim) {
      const int rel = c - g.gated_offset_in, u = rel / g.dim;
      float f, df;
      activation(g.act, row[g.gate_offset_in + u], f, df);
      v += g.cst * f * grow[g.offset_out + rel];
    }
    if (c >= g.gate_offset_in && c < g.gate_offset_in + g.mul) {
      const int u = c - g.gate_offset_in;
      float f, df;
      activation(g.act, row[c], f, df);
      float s = 0.f;
      for (int m = 0; m < g.dim; ++m) s += grow[g.offset_out + u * g.dim + m] * row[g.gated_offset_in + u * g.dim + m];
      v += g.cst * df * s;
    }
  }
  gx[id] = v;
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
  if (dtype != E3X_F32) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_forward: only fp32 storage is implemented");
  Tables t;
  int rc = fill_tables("e3x_gate_forward", acts, n_acts, gates, n_gates, in_dim, out_dim, &t);
  if (rc) return rc;
  if (Z < 0) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_forward: negative batch");
  if (Z == 0 || out_dim == 0) return E3X_OK;
  if (!x || !out) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_forward: null pointer");
  const long long n = Z * out_dim, blocks = (n + 255) / 256;
  if (blocks >= (1LL << 31)) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_forward: too many elements for one launch");
  hipLaunchKernelGGL(gate_fwd_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, t, (const float*)x,
                     (float*)out, (long long)Z, (int)in_dim, (int)out_dim);
  if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_gate_forward: kernel launch failed");
  return E3X_OK;
}

extern "C" int e3x_gate_backward(const e3x_act_block* acts, int32_t n_acts, const e3x_gate_block* gates, int32_t n_gates,
                                 const void* x, const void* grad_out, void* grad_x, int64_t Z, int64_t in_dim,
                                 int64_t out_dim, int32_t dtype, void* stream) {
  if (dtype != E3X_F32) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward: only fp32 storage is implemented");
  Tables t;
  int rc = fill_tables("e3x_gate_backward", acts, n_acts, gates, n_gates, in_dim, out_dim, &t);
  if (rc) return rc;
  if (Z < 0) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward: negative batch");
  if (Z == 0 || in_dim == 0) return E3X_OK;
  if (!x || !grad_out || !grad_x) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward: null pointer");
  const long long n = Z * in_dim, blocks = (n + 255) / 256;
  if (blocks >= (1LL << 31)) return e3x::fail(E3X_ERR_INVALID, "e3x_gate_backward: too many elements for one launch");
  hipLaunchKernelGGL(gate_bwd_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, t, (const float*)x,
                     (const float*)grad_out, (float*)grad_x, (long long)Z, (int)in_dim, (int)out_dim);
  if (hipGetLastError() != hipSuccess) return e3x::fail(E3X_ERR_HIP, "e3x_gate_backward: kernel launch failed");
  return E3X_OK;
}
