// Fused fully-connected network of scalars (the radial network of a convolution): plan creation,
// emission of the constexpr tables that specialise templates/fc_mfma.inc, code-object loading, launches.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "e3x_internal.h"
#include "jit.h"

namespace {
constexpr int kMaxDevices = 64;
constexpr int kMaxLayers = 8;
// LDS the packed weights may take (the CU has 160 KB; leave room for the runtime's own use)
constexpr int64_t kMaxPackedBytes = 150 * 1024;
// registers of a lane that may hold activations (of 256 at two waves per SIMD): the input and output of a hidden
// layer, width / 2 registers each per 32 rows, are live together
constexpr int kMaxLiveRegs = 192;
}  // namespace

struct e3x_fc_plan {
  std::vector<int> hs, hp;
  int n_layers = 0, rows_per_wg = 0, waves = 8;
  bool epilogue = false;  // outputs are multiplied by an activation derivative of a caller-supplied tensor
  int input_act = 0;      // the rows given are pre-activations: the network starts from input_cst * act(x)
  double input_cst = 1.0;
  int64_t packed_numel = 0;   // floats of the packed network (a split layer takes 1.5 per weight)
  int64_t logical_numel = 0;  // weights of the padded network
  std::string key, hsaco;
  std::mutex mu;
  hipModule_t module[kMaxDevices] = {nullptr};
  hipFunction_t fn_pack[kMaxDevices] = {nullptr};
  hipFunction_t fn_fwd[kMaxDevices] = {nullptr};
  int n_cu[kMaxDevices] = {0};
  // weight gradient of a one-layer plan: a code object of its own, built on first use
  double scale0 = 1.0;  // factor on x @ W of the first layer
  int dw_col_groups = 0;
  std::string dw_key, dw_hsaco;
  hipModule_t dw_module[kMaxDevices] = {nullptr};
  hipFunction_t fn_dw[kMaxDevices] = {nullptr};
};

namespace {

using e3x::fail;

std::string fstr(double v) {
  char buf[64];
  std::snprintf(buf, sizeof(buf), "%.9ef", v);
  return buf;
}

int round_up(int v, int m) { return (v + m - 1) / m * m; }

bool env_split() {
  const char* v = std::getenv("E3X_FC_SPLIT");
  return !(v && v[0] == '0');
}

bool env_split_wide() {
  const char* v = std::getenv("E3X_FC_SPLIT_WIDE");
  return !(v && v[0] == '0');
}

int load_functions(e3x_fc_plan* P, int dev) {
  std::lock_guard<std::mutex> lock(P->mu);
  if (P->module[dev]) return E3X_OK;
  hipModule_t mod = nullptr;
  hipError_t err = hipModuleLoad(&mod, P->hsaco.c_str());
  if (err != hipSuccess) return fail(E3X_ERR_HIP, "hipModuleLoad(" + P->hsaco + ") failed: " + hipGetErrorString(err));
  if (hipModuleGetFunction(&P->fn_pack[dev], mod, "e3x_fc_pack") != hipSuccess ||
      hipModuleGetFunction(&P->fn_fwd[dev], mod, "e3x_fc_forward_k") != hipSuccess)
    return fail(E3X_ERR_HIP, "kernels missing from " + P->hsaco);
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
  P->n_cu[dev] = n;
  P->module[dev] = mod;
  return E3X_OK;
}

}  // namespace

extern "C" int e3x_fc_plan_create(const int32_t* hs, int32_t n_hs, int32_t act, double act_cst, int32_t out_act,
                                  double variance_in, double variance_out, int32_t dtype, e3x_fc_plan** out) {
  return e3x_fc_plan_create_fused(hs, n_hs, act, act_cst, out_act, variance_in, variance_out, dtype, E3X_ACT_IDENTITY, 1.0,
                                  E3X_ACT_IDENTITY, 1.0, out);
}

extern "C" int e3x_fc_plan_create_fused(const int32_t* hs, int32_t n_hs, int32_t act, double act_cst, int32_t out_act,
                                        double variance_in, double variance_out, int32_t dtype, int32_t input_act,
                                        double input_cst, int32_t epilogue_act, double epilogue_cst, e3x_fc_plan** out) {
  if (!hs || !out) return fail(E3X_ERR_INVALID, "e3x_fc_plan_create: null argument");
  if (epilogue_act < E3X_ACT_IDENTITY || epilogue_act > E3X_ACT_RELU || input_act < E3X_ACT_IDENTITY || input_act > E3X_ACT_RELU)
    return fail(E3X_ERR_INVALID, "e3x_fc_plan_create: unknown input or epilogue activation");
  if (dtype != E3X_F32) return fail(E3X_ERR_INVALID, "e3x_fc_plan_create: only fp32 storage is implemented");
  if (n_hs < 2 || n_hs - 1 > kMaxLayers) return fail(E3X_ERR_INVALID, "e3x_fc_plan_create: 1 to 8 layers");
  if (act < E3X_ACT_IDENTITY || act > E3X_ACT_RELU) return fail(E3X_ERR_INVALID, "e3x_fc_plan_create: unknown activation");
  if (!(variance_in > 0) || !(variance_out > 0)) return fail(E3X_ERR_INVALID, "e3x_fc_plan_create: variances must be positive");
  const int NL = n_hs - 1;
  std::unique_ptr<e3x_fc_plan> P(new e3x_fc_plan);
  P->n_layers = NL;
  for (int i = 0; i <= NL; ++i) {
    if (hs[i] < 1 || hs[i] > (1 << 20)) return fail(E3X_ERR_INVALID, "e3x_fc_plan_create: bad layer width");
    P->hs.push_back(hs[i]);
    P->hp.push_back(round_up(hs[i], i == 0 ? 8 : 32));
  }
  for (int l = 0; l < NL; ++l) P->logical_numel += (int64_t)P->hp[l] * P->hp[l + 1];
  P->packed_numel = P->logical_numel;
  if (P->packed_numel * 4 > kMaxPackedBytes)
    return fail(E3X_ERR_INVALID, "e3x_fc_plan_create: the weights of the network do not fit the LDS of a compute unit");
  // Layers with a narrow input (<= 64, the three bf16 images of the input cost 3/4 of its width in registers) and at
  // least four output tiles run as six bf16 matrix products (fp32-accurate, 3/8 of the matrix time) while the packed
  // network (6 bytes per weight of such a layer) still fits the LDS; the widest first.
  std::vector<int> split(NL, 0);
  if (env_split()) {
    std::vector<int> order;
    for (int l = 0; l < NL; ++l)
      if (P->hp[l] % 16 == 0 && P->hp[l] >= 32 && P->hp[l] <= 64 && P->hp[l + 1] >= 128) order.push_back(l);
    // a last layer from a wide input to at most 64 outputs (the input gradient of the layers above): its input is
    // split 16 columns at a time inside the loop, so the register cost does not grow with the width
    if (env_split_wide() && P->hp[NL - 1] % 16 == 0 && P->hp[NL - 1] > 64 && P->hp[NL] <= 64) order.push_back(NL - 1);
    std::sort(order.begin(), order.end(), [&](int a, int b) { return (int64_t)P->hp[a] * P->hp[a + 1] > (int64_t)P->hp[b] * P->hp[b + 1]; });
    for (int l : order) {
      const int64_t extra = (int64_t)P->hp[l] * P->hp[l + 1] / 2;
      if ((P->packed_numel + extra) * 4 <= kMaxPackedBytes) split[l] = 1, P->packed_numel += extra;
    }
  }

  // e3nn/nn/_fc.py:70-88: every layer but the last is followed by act (unit second moment: cst * act) and has
  // var_out = 1; the last has var_out = variance_out and act only with out_act.  _fc.py:38-48: with act,
  // act(x @ W / sqrt(h_in var_in)) * sqrt(var_out); without, x @ W / sqrt(h_in var_in / var_out).
  std::vector<double> wscale(NL);
  std::vector<int> acts(NL);
  double post_prev = 1.0, var_in = variance_in, out_post = 1.0;
  for (int l = 0; l < NL; ++l) {
    const bool last = l == NL - 1;
    const double var_out = last ? variance_out : 1.0;
    const bool has_act = act != E3X_ACT_IDENTITY && (!last || out_act);  // E3X_ACT_IDENTITY: act=None
    acts[l] = has_act ? act : E3X_ACT_IDENTITY;
    double post;
    if (has_act) {
      wscale[l] = post_prev / std::sqrt((double)hs[l] * var_in);
      post = act_cst * std::sqrt(var_out);
    } else {
      wscale[l] = post_prev / std::sqrt((double)hs[l] * var_in / var_out);
      post = 1.0;
    }
    if (last) out_post = post;
    if (l == 0) P->scale0 = wscale[0];
    post_prev = post;
    var_in = var_out;
  }

  // a wave carries 32 rs rows: the input and output activations of a hidden layer are live together
  // (rs (hp[l] + hp[l+1]) / 2 registers) next to rs accumulator tiles of 16
  int live = P->hp[NL - 1] / 2;
  for (int l = 0; l + 1 < NL; ++l) live = std::max(live, (P->hp[l] + P->hp[l + 1]) / 2);
  if (live > kMaxLiveRegs)
    return fail(E3X_ERR_INVALID, "e3x_fc_plan_create: layers too wide for the fused kernel (input or hidden width above 384, "
                                 "or two consecutive ones above 384 in total)");
  int rs = 2 * live + 32 + 24 <= 224 ? 2 : 1;
  int waves = 8;
  if (const char* v = std::getenv("E3X_FC_RS")) rs = std::atoi(v);
  if (const char* v = std::getenv("E3X_FC_WAVES")) waves = std::atoi(v);
  if ((rs != 1 && rs != 2) || waves < 1 || waves > 16) return fail(E3X_ERR_INVALID, "E3X_FC_RS must be 1 or 2, E3X_FC_WAVES 1..16");
  P->waves = waves;
  P->rows_per_wg = waves * 32 * rs;
  std::ostringstream s;
  s << "// generated: one fully-connected network\n#include <stdint.h>\nnamespace cfg {\n";
  s << "constexpr int NL = " << NL << ";\nconstexpr int H[NL + 1] = {";
  for (int i = 0; i <= NL; ++i) s << (i ? ", " : "") << P->hs[i];
  s << "};\nconstexpr int HP[NL + 1] = {";
  for (int i = 0; i <= NL; ++i) s << (i ? ", " : "") << P->hp[i];
  s << "};\nconstexpr int ACT[NL] = {";
  for (int l = 0; l < NL; ++l) s << (l ? ", " : "") << acts[l];
  s << "};\nconstexpr bool SPLITL[NL] = {";
  for (int l = 0; l < NL; ++l) s << (l ? ", " : "") << (split[l] ? "true" : "false");
  s << "};\nconstexpr float WSCALE[NL] = {";
  for (int l = 0; l < NL; ++l) s << (l ? ", " : "") << fstr(wscale[l]);
  s << "};\nconstexpr float OUT_POST = " << fstr(out_post) << ";\n";
  s << "constexpr int EPI_ACT = " << epilogue_act << ";\nconstexpr float EPI_CST = " << fstr(epilogue_cst) << ";\n";
  s << "constexpr int IN_ACT = " << input_act << ";\nconstexpr float IN_CST = " << fstr(input_cst) << ";\n";
  P->epilogue = epilogue_act != E3X_ACT_IDENTITY;
  P->input_act = input_act;
  P->input_cst = input_cst;
  s << "constexpr int RS = " << rs << ", WAVES = " << waves << ";\n}  // namespace cfg\n";
  if (const char* v = std::getenv("E3X_FC_STREAM")) s << "#define E3X_FC_STREAM " << std::atoi(v) << "\n";
  if (const char* v = std::getenv("E3X_FC_STREAM_DIST")) s << "#define E3X_FC_STREAM_DIST " << std::max(1, std::atoi(v)) << "\n";
  const std::string src = s.str() + e3x::kTplCommon + e3x::kTplFcMfma;
  int rc = e3x::get_code_object("fc_mfma", src, &P->key, &P->hsaco);
  if (rc) return rc;
  *out = P.release();
  return E3X_OK;
}

extern "C" int e3x_fc_plan_destroy(e3x_fc_plan* plan) {
  delete plan;  // code objects stay loaded for the life of the process
  return E3X_OK;
}

extern "C" int e3x_fc_plan_prepare_backward_w(e3x_fc_plan* P) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_fc_plan_prepare_backward_w: null plan");
  if (P->n_layers != 1) return fail(E3X_ERR_INVALID, "e3x_fc_backward_w: one-layer plans only");
  std::lock_guard<std::mutex> lock(P->mu);
  if (!P->dw_hsaco.empty()) return E3X_OK;
  const int mt = (P->hs[0] + 31) / 32, nt = (P->hs[1] + 31) / 32;
  if (mt > 8) return fail(E3X_ERR_INVALID, "e3x_fc_backward_w: input width above 256");
  int ntw = std::min((nt + 3) / 4, std::max(1, 10 / mt));  // <= 160 accumulator registers per lane
  P->dw_col_groups = (nt + 4 * ntw - 1) / (4 * ntw);
  std::ostringstream s;
  s << "// generated: weight gradient of one dense layer\n#include <stdint.h>\n";
  if (const char* v = std::getenv("E3X_FCDW_KU")) s << "#define E3X_FCDW_KU " << std::atoi(v) << "\n";
  if (const char* v = std::getenv("E3X_FCDW_OCC")) s << "#define E3X_FCDW_OCC " << std::atoi(v) << "\n";
  if (const char* v = std::getenv("E3X_FCDW_SPLIT")) s << "#define E3X_FCDW_SPLIT " << std::atoi(v) << "\n";
  if (const char* v = std::getenv("E3X_FCDW_SHARE")) s << "#define E3X_FCDW_SHARE " << std::atoi(v) << "\n";
  s << "namespace cfg {\n";
  s << "constexpr int H_IN = " << P->hs[0] << ", H_OUT = " << P->hs[1] << ", NTW = " << ntw << ";\n";
  s << "constexpr float SCALE = " << fstr(P->scale0) << ";\n";
  s << "constexpr int IN_ACT = " << P->input_act << ";\nconstexpr float IN_CST = " << fstr(P->input_cst) << ";\n}  // namespace cfg\n";
  const std::string src = s.str() + e3x::kTplCommon + e3x::kTplFcDw;
  return e3x::get_code_object("fc_dw", src, &P->dw_key, &P->dw_hsaco);
}

extern "C" int e3x_fc_backward_w(e3x_fc_plan* P, const void* x, const void* grad_out, void* grad_w, int64_t Z, void* stream) {
  int rc = e3x_fc_plan_prepare_backward_w(P);
  if (rc) return rc;
  if (Z < 0) return fail(E3X_ERR_INVALID, "e3x_fc_backward_w: negative batch");
  if (!grad_w || (Z > 0 && (!x || !grad_out))) return fail(E3X_ERR_INVALID, "e3x_fc_backward_w: null pointer");
  hipStream_t st = (hipStream_t)stream;
  if ((rc = e3x::fill_zero_bytes(grad_w, (size_t)P->hs[0] * P->hs[1] * 4, stream))) return rc;
  if (Z == 0) return E3X_OK;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(E3X_ERR_HIP, "hipGetDevice failed");
  {
    std::lock_guard<std::mutex> lock(P->mu);
    if (!P->dw_module[dev]) {
      hipModule_t mod = nullptr;
      hipError_t err = hipModuleLoad(&mod, P->dw_hsaco.c_str());
      if (err != hipSuccess) return fail(E3X_ERR_HIP, "hipModuleLoad(" + P->dw_hsaco + ") failed: " + hipGetErrorString(err));
      if (hipModuleGetFunction(&P->fn_dw[dev], mod, "e3x_fc_dw_k") != hipSuccess)
        return fail(E3X_ERR_HIP, "kernel e3x_fc_dw_k missing from " + P->dw_hsaco);
      P->dw_module[dev] = mod;
    }
  }
  // two workgroups per compute unit (over all column groups) share the rows in trips of 16
  int per_cu = 2;
  if (const char* v = std::getenv("E3X_FCDW_OCC")) per_cu = std::atoi(v);
  long long slices = std::max(1, 256 * per_cu / P->dw_col_groups);
  slices = std::min<long long>(slices, (Z + 255) / 256);
  long long n_rows = Z;
  void* args[] = {&x, &grad_out, &grad_w, &n_rows};
  hipError_t err = hipModuleLaunchKernel(P->fn_dw[dev], (unsigned)slices, (unsigned)P->dw_col_groups, 1, 256, 1, 1, 0, st, args,
                                         nullptr);
  if (err != hipSuccess) return fail(E3X_ERR_HIP, std::string("e3x_fc_backward_w: launch failed: ") + hipGetErrorString(err));
  return E3X_OK;
}

extern "C" size_t e3x_fc_workspace_bytes(const e3x_fc_plan* P) { return P ? (size_t)P->packed_numel * 4 : 0; }

extern "C" const char* e3x_fc_plan_key(const e3x_fc_plan* P) { return P ? P->key.c_str() : ""; }

extern "C" int e3x_fc_forward(e3x_fc_plan* P, const void* x, const void* const* weights, void* out, int64_t Z,
                              void* workspace, size_t workspace_bytes, void* stream) {
  return e3x_fc_forward_epilogue(P, x, weights, nullptr, out, Z, workspace, workspace_bytes, stream);
}

extern "C" int e3x_fc_forward_epilogue(e3x_fc_plan* P, const void* x, const void* const* weights, const void* z, void* out,
                                       int64_t Z, void* workspace, size_t workspace_bytes, void* stream) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_fc_forward: null plan");
  if (P->epilogue && !z && Z > 0)
    return fail(E3X_ERR_INVALID, "e3x_fc_forward: this plan multiplies by an activation derivative and needs z "
                                 "(e3x_fc_forward_epilogue)");
  if (!P->epilogue) z = nullptr;
  if (Z < 0) return fail(E3X_ERR_INVALID, "e3x_fc_forward: negative batch");
  if (Z == 0) return E3X_OK;
  if (!x || !out || !weights || !workspace) return fail(E3X_ERR_INVALID, "e3x_fc_forward: null pointer");
  if (workspace_bytes < (size_t)P->packed_numel * 4) return fail(E3X_ERR_INVALID, "e3x_fc_forward: workspace too small");
  if (((uintptr_t)workspace & 15) || ((uintptr_t)x & 15))
    return fail(E3X_ERR_INVALID, "e3x_fc_forward: x and workspace must be 16-byte aligned");
  struct {
    const void* w[8];
  } ptrs = {};
  for (int l = 0; l < P->n_layers; ++l) {
    if (!weights[l]) return fail(E3X_ERR_INVALID, "e3x_fc_forward: null weight pointer");
    ptrs.w[l] = weights[l];
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(E3X_ERR_HIP, "hipGetDevice failed");
  int rc = load_functions(P, dev);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  {
    void* args[] = {&ptrs, &workspace};
    hipError_t err = hipModuleLaunchKernel(P->fn_pack[dev], (unsigned)((P->logical_numel + 255) / 256), 1, 1, 256, 1, 1, 0, st,
                                           args, nullptr);
    if (err != hipSuccess) return fail(E3X_ERR_HIP, std::string("e3x_fc_forward: pack launch failed: ") + hipGetErrorString(err));
  }
  long long n_rows = Z;
  long long tiles = (Z + P->rows_per_wg - 1) / P->rows_per_wg;
  long long blocks = tiles < P->n_cu[dev] ? tiles : P->n_cu[dev];  // one persistent workgroup per compute unit
  void* args[] = {&x, &workspace, &out, &n_rows, &z};
  hipError_t err = hipModuleLaunchKernel(P->fn_fwd[dev], (unsigned)blocks, 1, 1, 64 * P->waves, 1, 1, 0, st, args, nullptr);
  if (err != hipSuccess) return fail(E3X_ERR_HIP, std::string("e3x_fc_forward: launch failed: ") + hipGetErrorString(err));
  return E3X_OK;
}
