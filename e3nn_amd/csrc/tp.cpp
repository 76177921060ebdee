// Tensor-product plans: validation of an instruction set, emission of the constexpr
// tables that specialise the device templates, code-object loading and kernel launches.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "e3x_internal.h"
#include "jit.h"

namespace {

struct PathInfo {
  int in1, in2, out, mode, has_w;
  double pw;
  int woff;  // offset in the flat weight vector (weighted paths only)
};

constexpr int kMaxDevices = 64;

}  // namespace

// One compiled code object.  A plan is usually one kernel; large uvu instruction sets are split
// into several kernels over disjoint output irreps so that each keeps its accumulators in registers.
struct SubKernel {
  std::string key, hsaco;
  std::vector<int> path_ids;  // indices into e3x_plan::paths
  int lanes = 64, chunks = 1, upl = 1, waves_per_block = 4;
  bool cached_weights = false;  // uvw_small: weights in registers, rows walked with a grid-sized stride
  hipModule_t module[kMaxDevices] = {nullptr};
  hipFunction_t fn_plain[kMaxDevices] = {nullptr};
  hipFunction_t fn_fused[kMaxDevices] = {nullptr};
  hipFunction_t fn_bwd_edge[kMaxDevices] = {nullptr};
  hipFunction_t fn_bwd_edge_lds[kMaxDevices] = {nullptr};  // the variant with every row through LDS, when generated
  bool bwd_lds = false;
  hipFunction_t fn_dw[kMaxDevices] = {nullptr};
  hipFunction_t fn_pack[kMaxDevices] = {nullptr};
  // uvu: the edge-parallel backward kernel is a code object of its own (other lane layout), built on first use
  std::unique_ptr<SubKernel> bwd;
  // uvu, transposed plan of a message step: the fused kernel that also writes the weight gradient, built on first use
  std::unique_ptr<SubKernel> fused_dw;
  hipFunction_t fn_fused_dw[kMaxDevices] = {nullptr};
  hipFunction_t fn_fused_dw_x2[kMaxDevices] = {nullptr};  // ... and the gradient of the second input
};

struct e3x_plan {
  std::vector<e3x_irrep> in1, in2, out;
  std::vector<int> off1, off2, offo;
  std::vector<PathInfo> paths;
  int shared_weights = 1, dtype = E3X_F32;
  int64_t in1_dim = 0, in2_dim = 0, out_dim = 0, weight_numel = 0;
  std::string family, key;
  // which instruction forms the products, forward and in the uvw weight gradient (the latter once that kernel is built)
  std::string arithmetic = "fp32 vector ALU", arithmetic_dw;
  bool zero_fill = false;  // some output irrep is reached by no instruction
  int n_targets = 0;       // uvw_mfma: grid.y
  std::vector<int> node_tile_rows;  // uvw_node: rows per workgroup of each target, in grid order
  // uvu: the message kernel with the radial network inside, one per network description, built on first use
  std::vector<std::unique_ptr<SubKernel>> radial;
  std::vector<std::unique_ptr<SubKernel>> radial_retired;  // kernels of earlier network descriptions: a launch may still hold them
  std::string radial_desc;
  std::mutex mu;
  std::vector<std::unique_ptr<SubKernel>> subs;
  // uvu with the spherical harmonics 0 .. lmax as second input: variants of the kernels of `subs` that form the
  // harmonics from the edge vectors themselves, per (normalize, normalization), built on first use
  std::map<int, std::vector<std::unique_ptr<SubKernel>>> sh_subs;
  // uvu, bf16 storage: the message kernel (gather + product + scatter) with the contraction on the matrix cores,
  // when the instruction set fits it; the plain product keeps the kernels of `subs`
  std::unique_ptr<SubKernel> msg_mfma;
  int msg_groups = 0;  // wavefronts per output row
  // uvw_mfma: the weight-gradient kernel is a code object of its own, built on first use
  std::unique_ptr<SubKernel> dw;
  long long dw_tiles = 0;  // grid.x: the largest tile count of a path
  int dw_paths = 0;        // grid.y
};

namespace {

using e3x::fail;

int dim_of(const e3x_irrep& r) { return r.mul * (2 * r.l + 1); }

int env_int(const char* name, int fallback) {
  const char* v = std::getenv(name);
  return (v && v[0]) ? std::atoi(v) : fallback;
}

std::string fstr(double v) {
  char buf[64];
  std::snprintf(buf, sizeof(buf), "%.9ef", v);
  return buf;
}

int pow2_at_least(int v, int lo) {
  int p = lo;
  while (p < v) p *= 2;
  return p;
}

// ---- common part of the generated tables ------------------------------------------
void emit_header(std::ostringstream& s, const e3x_plan& P, int lanes = 64, int chunks = 1) {
  s << "// generated: tables of one instruction set\n#include <stdint.h>\nnamespace cfg {\n";
  s << "typedef " << (P.dtype == E3X_BF16 ? "unsigned short" : "float") << " store_t;\n";
  s << "constexpr bool SHARED_W = " << (P.shared_weights ? "true" : "false") << ";\n";
  s << "constexpr int IN1_DIM = " << P.in1_dim << ", IN2_DIM = " << P.in2_dim << ", OUT_DIM = " << P.out_dim
    << ", W_NUMEL = " << P.weight_numel << ";\n";
  s << "constexpr int LANES = " << lanes << ", CHUNKS = " << chunks << ";\n";
}

struct NzList {
  std::vector<std::string> rows;
  std::vector<int> beg, end;
};

// non-zeros of pw * wigner_3j per path, as "{i, j, k, c}" rows
NzList emit_nz(const e3x_plan& P, const std::vector<int>& ids) {
  NzList L;
  for (int id : ids) {
    const auto& p = P.paths[id];
    const int l1 = P.in1[p.in1].l, l2 = P.in2[p.in2].l, l3 = P.out[p.out].l;
    const auto& C = e3x::wigner_3j(l1, l2, l3);
    const int d2 = 2 * l2 + 1, d3 = 2 * l3 + 1;
    L.beg.push_back((int)L.rows.size());
    for (int i = 0; i < 2 * l1 + 1; ++i)
      for (int j = 0; j < d2; ++j)
        for (int k = 0; k < d3; ++k) {
          const double c = C[(i * d2 + j) * d3 + k] * p.pw;
          if (c != 0.0) {
            std::ostringstream r;
            r << "{" << i << ", " << j << ", " << k << ", " << fstr(c) << "}";
            L.rows.push_back(r.str());
          }
        }
    L.end.push_back((int)L.rows.size());
  }
  return L;
}

void emit_nz_table(std::ostringstream& s, const NzList& L) {
  s << "struct Nz { int i, j, k; float c; };\n";
  s << "constexpr int N_NZ = " << L.rows.size() << ";\n";
  s << "constexpr Nz nz[N_NZ > 0 ? N_NZ : 1] = {\n";
  for (const auto& r : L.rows) s << "  " << r << ",\n";
  if (L.rows.empty()) s << "  {0, 0, 0, 0.f}\n";
  s << "};\n";
}

// ---- uvu ---------------------------------------------------------------------------

// Splits the paths into kernels over disjoint output irreps when one kernel would need too many
// accumulator registers: paths sharing an output stay together, groups are formed per input-1 irrep
// (so each kernel gathers only its own slice of the source row).
std::vector<std::vector<int>> split_uvu_paths(const e3x_plan& P, int acc_limit = 0) {
  std::vector<int> all(P.paths.size());
  for (size_t i = 0; i < all.size(); ++i) all[i] = (int)i;
  int acc = 0;
  std::vector<char> usedo(P.out.size(), 0);
  for (const auto& p : P.paths)
    if (!usedo[p.out]) { usedo[p.out] = 1; acc += 2 * P.out[p.out].l + 1; }
  // fp32: one kernel up to 128 accumulators per multiplicity index (measured faster on the 99-accumulator
  // MACE set than four kernels); bf16 storage is ALU-bound and prefers the smaller kernels
  const int limit = acc_limit > 0 ? acc_limit : (P.dtype == E3X_BF16 ? 48 : 128);
  int x1regs = 0;
  std::vector<char> used1(P.in1.size(), 0);
  for (const auto& p : P.paths)
    if (!used1[p.in1]) { used1[p.in1] = 1; x1regs += 2 * P.in1[p.in1].l + 1; }
  // (transposed plans of the backward pass have many input irreps instead of many outputs)
  const int want = acc_limit > 0 ? (acc > limit) : env_int("E3X_UVU_SPLIT", (acc > limit || x1regs > 64) ? 1 : 0);
  if (!want || P.paths.empty()) return {all};
  // an output irrep fed from several input-1 irreps ties those inputs together
  std::vector<int> group_of_in1(P.in1.size());
  for (size_t a = 0; a < group_of_in1.size(); ++a) group_of_in1[a] = (int)a;
  auto find = [&](int a) { while (group_of_in1[a] != a) a = group_of_in1[a]; return a; };
  std::vector<int> first_in1(P.out.size(), -1);
  for (const auto& p : P.paths) {
    if (first_in1[p.out] < 0) first_in1[p.out] = p.in1;
    else group_of_in1[find(p.in1)] = find(first_in1[p.out]);
  }
  std::vector<std::vector<int>> parts;
  std::vector<int> part_of_group(P.in1.size(), -1);
  for (size_t i = 0; i < P.paths.size(); ++i) {
    const int gsel = find(P.paths[i].in1);
    if (part_of_group[gsel] < 0) { part_of_group[gsel] = (int)parts.size(); parts.emplace_back(); }
    parts[part_of_group[gsel]].push_back((int)i);
  }
  return parts;
}

// extra_cfg: more constants for the generated namespace; tpl: the device template to specialise (default: uvu.inc)
int build_uvu_source(e3x_plan& P, SubKernel& K, std::string* src, bool bwd_only = false, const std::string* extra_cfg = nullptr,
                     const char* tpl = nullptr) {
  int max_mul = 1;
  std::vector<char> used1(P.in1.size(), 0), usedo(P.out.size(), 0);
  long long unrolled = 0;
  for (int id : K.path_ids) {
    const auto& p = P.paths[id];
    if (P.in1[p.in1].mul != P.out[p.out].mul)
      return fail(E3X_ERR_INVALID, "uvu instruction needs irreps_in1[i_in1].mul == irreps_out[i_out].mul");
    used1[p.in1] = 1;
    usedo[p.out] = 1;
    max_mul = std::max(max_mul, P.in1[p.in1].mul);
  }
  if (P.in2_dim > 64) return fail(E3X_ERR_INVALID, "uvu kernel: irreps_in2.dim > 64 is not supported");
  int x1regs = 0, accregs = 0, wregs = 0;
  for (size_t a = 0; a < P.in1.size(); ++a) if (used1[a]) x1regs += 2 * P.in1[a].l + 1;
  for (size_t c = 0; c < P.out.size(); ++c) if (usedo[c]) accregs += 2 * P.out[c].l + 1;
  for (int id : K.path_ids) if (P.paths[id].has_w) wregs += P.in2[P.paths[id].in2].mul;
  if (x1regs > 96) return fail(E3X_ERR_INVALID, "uvu kernel: more than 96 input components per multiplicity index");
  if (accregs > 256) return fail(E3X_ERR_INVALID, "uvu kernel: more than 256 output components per multiplicity index");
  // multiplicity indices per lane: 4 makes every per-lane access a 16-byte run; needs mul % 4 == 0
  // and a register budget of about 200 for one set of edge registers plus the accumulators
  int upl = 4;
  auto fits = [&](int u) {
    for (size_t a = 0; a < P.in1.size(); ++a) if (used1[a] && P.in1[a].mul % u) return false;
    if (P.dtype == E3X_BF16 && u == 4 && accregs > 24) return false;  // measured: 2 per lane is faster there
    return u * (accregs + x1regs + wregs) + (int)P.in2_dim <= 200;
  };
  while (upl > 1 && !fits(upl)) upl /= 2;
  // narrow sets: a group of lanes is at least 8 wide, so fewer indices per lane keep its lanes busy (measured on
  // 500 000 edges, l <= 2: multiplicity 8 with 4 / 2 / 1 per lane 0.203 / 0.109 / 0.096 ms in fp32 and 0.485 / 0.138 /
  // 0.085 ms in bf16 storage; multiplicity 16: 0.230 / 0.126 / 0.123 ms and 0.520 / 0.098 / 0.099 ms)
  while (upl > 1 && max_mul / upl < 8) upl /= 2;
  upl = env_int("E3X_UVU_UPL", upl);
  // the backward kernel also holds the output gradient of its indices: one index per lane keeps it at several waves
  // per SIMD (measured on the 32-channel l <= 2 set: 1.39 ms against 1.85 ms with four)
  // -- as long as a wavefront still covers every index of an edge (one chunk: grad_x2 needs no atomics then)
  if (bwd_only) {
    int b = 1;
    while (b < upl && (max_mul + b - 1) / b > 64) b *= 2;
    upl = env_int("E3X_UVU_BWD_UPL", b);
  }
  if (upl != 1 && upl != 2 && upl != 4) return fail(E3X_ERR_INVALID, "E3X_UVU_UPL must be 1, 2 or 4");
  for (size_t a = 0; a < P.in1.size(); ++a)
    if (used1[a] && P.in1[a].mul % upl) return fail(E3X_ERR_INVALID, "uvu kernel: multiplicity not divisible by UPL");
  const int lane_units = (max_mul + upl - 1) / upl;
  K.upl = upl;
  K.lanes = lane_units > 32 ? 64 : pow2_at_least(lane_units, 8);
  K.chunks = (lane_units + K.lanes - 1) / K.lanes;

  std::ostringstream s;
  emit_header(s, P, K.lanes, K.chunks);
  s << "constexpr int UPL = " << upl << ";\n";
  int reg = 0;
  s << "struct In1 { int off, d, mul, reg; bool used; };\n";
  s << "constexpr int N_IN1 = " << P.in1.size() << ";\nconstexpr In1 in1[N_IN1] = {\n";
  for (size_t a = 0; a < P.in1.size(); ++a) {
    const int d = 2 * P.in1[a].l + 1;
    s << "  {" << P.off1[a] << ", " << d << ", " << P.in1[a].mul << ", " << reg << ", " << (used1[a] ? "true" : "false")
      << "},\n";
    if (used1[a]) reg += d;
  }
  s << "};\nconstexpr int X1_REGS = " << reg << ";\n";
  reg = 0;
  s << "struct Out { int off, d, mul, reg; bool used; };\n";
  s << "constexpr int N_OUT = " << P.out.size() << ";\nconstexpr Out outs[N_OUT] = {\n";
  for (size_t c = 0; c < P.out.size(); ++c) {
    const int d = 2 * P.out[c].l + 1;
    s << "  {" << P.offo[c] << ", " << d << ", " << P.out[c].mul << ", " << reg << ", " << (usedo[c] ? "true" : "false")
      << "},\n";
    if (usedo[c]) reg += d;
  }
  s << "};\nconstexpr int ACC_REGS = " << reg << ";\n";
  NzList L = emit_nz(P, K.path_ids);
  int wreg = 0;
  s << "struct Path { int in1, x2off, d2, V, out, woff, wreg; bool has_w; int nz_beg, nz_end; };\n";
  s << "constexpr int N_PATH = " << K.path_ids.size() << ";\nconstexpr Path paths[N_PATH > 0 ? N_PATH : 1] = {\n";
  for (size_t i = 0; i < K.path_ids.size(); ++i) {
    const auto& p = P.paths[K.path_ids[i]];
    const int V = P.in2[p.in2].mul;
    s << "  {" << p.in1 << ", " << P.off2[p.in2] << ", " << 2 * P.in2[p.in2].l + 1 << ", " << V << ", " << p.out << ", "
      << p.woff << ", " << wreg << ", " << (p.has_w ? "true" : "false") << ", " << L.beg[i] << ", " << L.end[i]
      << "},\n";
    if (p.has_w) wreg += V;
    unrolled += (long long)V * (L.end[i] - L.beg[i]);
  }
  if (K.path_ids.empty()) s << "  {0, 0, 1, 0, 0, 0, 0, false, 0, 0}\n";
  s << "};\nconstexpr int W_REGS = " << wreg << ";\n";
  if (wreg > 128 || unrolled * upl > 40000)
    return fail(E3X_ERR_INVALID, "uvu kernel: instruction set too large to unroll (irreps_in2 multiplicities too high)");
  emit_nz_table(s, L);
  // two register sets (software prefetch of the next edge) while they fit a high-occupancy budget
  bool prefetch = upl * (accregs + 2 * (x1regs + wregs)) + 2 * (int)P.in2_dim <= 96;
  prefetch = env_int("E3X_UVU_PREFETCH", prefetch ? 1 : 0) != 0;
  s << "constexpr bool PREFETCH = " << (prefetch ? "true" : "false") << ";\n";
  K.waves_per_block = env_int("E3X_UVU_WAVES_PER_BLOCK", 4);
  s << "#define E3X_WAVES_PER_BLOCK " << K.waves_per_block << "\n";
  if (bwd_only) s << "#define E3X_UVU_BWD_ONLY 1\n";
  if (bwd_only) {
    // second kernel of the code object: the rows of an edge through LDS in 16-byte pieces (see the template); one
    // kernel and one chunk must cover the instruction set so that the group writes the whole weight-gradient row
    // at most 8 KB of LDS per wavefront: beyond that the row images cost more occupancy than the loads they replace
    // (measured with 1120-wide cotangent rows, 14 KB per wavefront, two waves per SIMD: 2.1 ms against 1.3 ms direct)
    const int groups = 64 / K.lanes;
    const int64_t lds = (int64_t)groups * (P.in1_dim + P.out_dim + P.weight_numel) * 4;
    K.bwd_lds = P.dtype == E3X_F32 && !P.shared_weights && K.chunks == 1 && K.path_ids.size() == P.paths.size() &&
                P.weight_numel > 0 && P.in1_dim > 0 && P.in1_dim % 4 == 0 && P.out_dim % 4 == 0 && P.weight_numel % 4 == 0 &&
                lds <= 8 * 1024 && env_int("E3X_UVU_BWD_LDS", 1) != 0;
    if (K.bwd_lds) s << "#define E3X_UVU_BWD_LDS 1\n";
  }
  // coefficient folded into the edge attribute (see accumulate_edge); measured on one GPU, old -> new: 32 channels
  // l <= 2 at four indices per lane 0.637 -> 0.635 ms (degree 354: 4.91 -> 4.84), 128 channels l <= 3 in bf16 storage
  // 1.60 -> 1.48 ms, in fp32 at two indices per lane 1.68 -> 1.77 ms
  const bool fold = env_int("E3X_UVU_FOLD", (upl == 4 || P.dtype == E3X_BF16) ? 1 : 0) != 0;
  if (fold) s << "#define E3X_UVU_FOLD 1\n";
  // All loads of an edge ahead of its first product (a scheduling barrier in the edge loop) while the operands of an
  // edge leave room for three waves per SIMD; measured: + 3 % on the 32-channel l <= 2 set, + 13 % in bf16 storage,
  // - 2 % on the 128-channel l <= 3 set in fp32, whose operands alone take ~150 registers.
  const bool loads_first = P.dtype == E3X_BF16 || upl * (accregs + x1regs + wregs) + (int)P.in2_dim <= 140;
  if (env_int("E3X_UVU_SCHED", loads_first ? 1 : 0) == 0) s << "#define E3X_UVU_SCHED 0\n";
  // The source row through LDS (see fetch_x1 / stage_x1 in the template): when a lane owns several indices of irreps
  // with d > 1, whose runs make the direct 16-byte loads touch d lines per lane group.  Needs whole 16-byte pieces.
  {
    const int epp = P.dtype == E3X_BF16 ? 8 : 4;
    bool whole = !bwd_only && !tpl && !prefetch && upl * (P.dtype == E3X_BF16 ? 2 : 4) % 16 == 0 && P.in1_dim % (epp * K.lanes) == 0;
    bool wide = false;
    for (size_t a = 0; a < P.in1.size(); ++a) {
      const int d = 2 * P.in1[a].l + 1;
      if (!used1[a] && P.in1[a].mul > 0) whole = false;  // split kernels gather only their own slice of the row
      if (used1[a] && (P.off1[a] % epp || (upl * d) % epp || P.in1[a].mul % upl || P.in1[a].mul > K.lanes * upl * K.chunks)) whole = false;
      wide = wide || (used1[a] && d > 1);
    }
    const long long lds = (long long)K.waves_per_block * (64 / K.lanes) * P.in1_dim * (P.dtype == E3X_BF16 ? 2 : 4);
    if (env_int("E3X_UVU_X1_LDS", (whole && wide && K.chunks == 1 && lds <= 49152) ? 1 : 0) && whole && K.chunks == 1 && lds <= 65536)
      s << "#define E3X_UVU_X1_LDS 1\n";
  }
  // The partial sums of the lane groups combined through LDS and the row stored as whole 16-byte pieces (see
  // reduce_store_row in the template): fp32, four indices per lane, several groups per wavefront, and a kernel that
  // owns the whole output row.  Measured on the 32-channel l <= 2 set: the shuffle butterfly and the 128-byte stores
  // it replaces were 15 % of the kernel.
  {
    bool ok = !bwd_only && !tpl && P.dtype == E3X_F32 && upl == 4 && K.lanes < 64 && K.chunks == 1 && P.out_dim % 4 == 0;
    for (size_t c = 0; c < P.out.size(); ++c) {
      if (P.out[c].mul == 0) continue;
      if (!usedo[c] || P.offo[c] % 4 || P.out[c].mul % 4 || P.out[c].mul > K.lanes * upl) ok = false;
    }
    const long long lds = (long long)K.waves_per_block * (64 / K.lanes) * P.out_dim * 4;
    if (ok && lds <= 49152 && env_int("E3X_UVU_LDS_REDUCE", 1)) s << "#define E3X_UVU_LDS_REDUCE 1\n";
  }
  if (extra_cfg) s << *extra_cfg;
  s << "}  // namespace cfg\n";
  *src = s.str() + e3x::kTplCommon + (tpl ? tpl : e3x::kTplUvu);
  return E3X_OK;
}


// ---- uvu message kernel on the matrix cores -----------------------------------------------------------------
// Tables of templates/uvu_mfma.inc.  Returns false (and builds nothing) when the instruction set does not fit:
// bf16 storage, per-edge weights on every instruction, multiplicity 1 on the second input, one multiplicity U = 128
// on the first input and the output, at most 16 components per multiplicity index on the first input, split over
// the two halves of the K range without cutting an irrep, and exactly one instruction per output irrep (the
// per-path output blocks that the reference's convolution builds, e3nn/nn/models/v2106/points_convolution.py:60-76).
bool build_uvu_msg_mfma_source(e3x_plan& P, SubKernel& K, std::string* src) {
  if (P.dtype != E3X_BF16 || P.shared_weights || P.paths.empty() || P.in2_dim > 16 || P.in2_dim == 0) return false;
  const int U = 128, UT = U / 32;
  std::vector<char> used1(P.in1.size(), 0);
  std::vector<int> n_out(P.out.size(), 0);
  for (const auto& p : P.paths) {
    if (p.mode != E3X_MODE_UVU || !p.has_w || P.in2[p.in2].mul != 1 || P.in1[p.in1].mul != U || P.out[p.out].mul != U)
      return false;
    used1[p.in1] = 1;
    if (++n_out[p.out] > 1) return false;
  }
  if (P.in1_dim % 8 || P.weight_numel % 8 || P.in2_dim % 8) return false;  // rows are read in 16-byte pieces
  // K slots: first-fit of the input irreps, largest first, into two halves of 8
  std::vector<int> order;
  for (size_t a = 0; a < P.in1.size(); ++a) if (used1[a]) order.push_back((int)a);
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return P.in1[a].l > P.in1[b].l; });
  std::vector<int> half_of(P.in1.size(), -1), slot0(P.in1.size(), 0);
  int fill[2] = {0, 0};
  std::vector<int> runs[2];
  for (int a : order) {
    const int d = 2 * P.in1[a].l + 1;
    const int h = fill[0] + d <= 8 ? 0 : (fill[1] + d <= 8 ? 1 : -1);
    if (h < 0) return false;
    half_of[a] = h, slot0[a] = fill[h], fill[h] += d;
    runs[h].push_back(a);
  }
  std::ostringstream s;
  emit_header(s, P);
  int prefetch = env_int("E3X_UVUM_PREFETCH", 2), mblk = env_int("E3X_UVUM_MBLK", 8);
  if (prefetch != 2 && prefetch != 4 && prefetch != 8) prefetch = 4;
  if (mblk != 8 && mblk != 16 && mblk != 32) mblk = 8;
  s << "constexpr int U = " << U << ", UT = " << UT << ", MBLK = " << mblk << ", PREFETCH = " << prefetch << ";\n";
  s << "#define E3X_UVUM_OCC " << env_int("E3X_UVUM_OCC", 3) << "\n";
  // K slot sl (0-7: first half, 8-15: second) of index u is component kslot_off[sl] + u * kslot_d[sl] of a source row
  int ks_off[16], ks_d[16];
  for (int i = 0; i < 16; ++i) ks_off[i] = 0, ks_d[i] = 0;
  for (int h = 0; h < 2; ++h)
    for (int a : runs[h]) {
      const int d = 2 * P.in1[a].l + 1;
      for (int i = 0; i < d; ++i) ks_off[8 * h + slot0[a] + i] = P.off1[a] + i, ks_d[8 * h + slot0[a] + i] = d;
    }
  s << "constexpr int kslot_off[16] = {";
  for (int i = 0; i < 16; ++i) s << ks_off[i] << ", ";
  s << "};\nconstexpr int kslot_d[16] = {";
  for (int i = 0; i < 16; ++i) s << ks_d[i] << ", ";
  s << "};\n";
  // paths and their Clebsch-Gordan non-zeros (path weight folded in)
  std::vector<int> all(P.paths.size());
  for (size_t i = 0; i < all.size(); ++i) all[i] = (int)i;
  NzList L = emit_nz(P, all);
  s << "struct GPath { int x2off, d2, half, slot0, d1, woff, ooff, d3, nz_beg, nz_end; };\n";
  s << "constexpr int NP = " << P.paths.size() << ";\nconstexpr GPath gpaths[NP] = {\n";
  for (size_t i = 0; i < P.paths.size(); ++i) {
    const auto& p = P.paths[i];
    s << "  {" << P.off2[p.in2] << ", " << 2 * P.in2[p.in2].l + 1 << ", " << half_of[p.in1] << ", " << slot0[p.in1] << ", "
      << 2 * P.in1[p.in1].l + 1 << ", " << p.woff << ", " << P.offo[p.out] << ", " << 2 * P.out[p.out].l + 1 << ", "
      << L.beg[i] << ", " << L.end[i] << "},\n";
  }
  s << "};\n";
  emit_nz_table(s, L);
  // matrix rows: the columns (path, k) of the product in pairs (k, k + 1) of one path, 16 pairs per 32-row tile,
  // two tiles per group (one wavefront per output row and group)
  struct PairRow { int path, k0, k1; };
  std::vector<PairRow> pr;
  for (size_t i = 0; i < P.paths.size(); ++i) {
    const int d3 = 2 * P.out[P.paths[i].out].l + 1;
    for (int k = 0; k < d3; k += 2) pr.push_back({(int)i, k, k + 1 < d3 ? k + 1 : -1});
  }
  // tiles per group: one keeps a wavefront at 64 accumulators and three waves per SIMD
  const int tiles = env_int("E3X_UVUM_TILES", 1) == 2 ? 2 : 1, ppg = 16 * tiles;
  const int ng = ((int)pr.size() + ppg - 1) / ppg;
  if (ng > 8) return false;  // one wavefront per group, one workgroup per output row
  K.waves_per_block = ng;
  while ((int)pr.size() < ng * ppg) pr.push_back({-1, -1, -1});
  s << "constexpr int TILES = " << tiles << ", NG = " << ng << ";\nstruct Pair { int path, k0, k1; };\nconstexpr Pair pairs[NG * "
    << ppg << "] = {\n";
  for (const auto& q : pr) s << "  {" << q.path << ", " << q.k0 << ", " << q.k1 << "},\n";
  s << "};\n";
  std::ostringstream gb, ge, rv, rh;
  int gw_max = 0;
  for (int g = 0; g < ng; ++g) {
    int lo = 1 << 30, hi = -1;
    unsigned valid[2] = {0, 0}, half[2] = {0, 0};
    for (int q = 0; q < ppg; ++q) {
      const PairRow& r = pr[g * ppg + q];
      if (r.path < 0) continue;
      lo = std::min(lo, r.path), hi = std::max(hi, r.path);
      const int tile = q / 16, row0 = 8 * ((q % 16) / 4) + (q % 16) % 4;
      const unsigned hb = (unsigned)half_of[P.paths[r.path].in1];
      valid[tile] |= 1u << row0, half[tile] |= hb << row0;
      if (r.k1 >= 0) valid[tile] |= 1u << (row0 + 4), half[tile] |= hb << (row0 + 4);
    }
    gb << lo << ", ", ge << hi + 1 << ", ";
    gw_max = std::max(gw_max, hi + 1 - lo);
    rv << "{" << valid[0] << "u" << (tiles == 2 ? ", " + std::to_string(valid[1]) + "u" : "") << "}, ";
    rh << "{" << half[0] << "u" << (tiles == 2 ? ", " + std::to_string(half[1]) + "u" : "") << "}, ";
  }
  s << "constexpr int gp_beg[NG] = {" << gb.str() << "};\nconstexpr int gp_end[NG] = {" << ge.str() << "};\n";
  s << "constexpr int GW_MAX = " << gw_max << ";\n";
  s << "constexpr unsigned row_valid[NG][TILES] = {" << rv.str() << "};\nconstexpr unsigned row_half[NG][TILES] = {" << rh.str() << "};\n";
  s << "}  // namespace cfg\n";
  P.msg_groups = ng;
  *src = s.str() + e3x::kTplCommon + e3x::kTplUvuMfma;
  return true;
}

// ---- uvw (lane <-> output multiplicity, VALU) ----------------------------------------
int build_uvw_small_source(e3x_plan& P, SubKernel& K, std::string* src) {
  int max_mul = 1;
  std::vector<char> usedo(P.out.size(), 0);
  bool all_uvw = true;
  for (const auto& p : P.paths) {
    usedo[p.out] = 1;
    max_mul = std::max(max_mul, P.out[p.out].mul);
    all_uvw = all_uvw && p.mode == E3X_MODE_UVW;
  }
  K.lanes = max_mul > 32 ? 64 : pow2_at_least(max_mul, 16);
  // long input rows: fewer rows per wavefront so that the staged rows fit in LDS (lanes beyond the output
  // multiplicity idle)
  while (K.lanes < 64 && (P.in1_dim + P.in2_dim) * 16 * (64 / K.lanes) > 65536) K.lanes *= 2;
  K.chunks = (max_mul + K.lanes - 1) / K.lanes;
  if ((P.in1_dim + P.in2_dim) * 16 * (64 / K.lanes) > 65536)
    return fail(E3X_ERR_INVALID, "uvw kernel: input rows too long for the LDS staging buffer");
  std::ostringstream s;
  emit_header(s, P, K.lanes, K.chunks);
  int reg = 0;
  s << "struct Out { int off, d, mul, reg; bool used; };\n";
  s << "constexpr int N_OUT = " << P.out.size() << ";\nconstexpr Out outs[N_OUT] = {\n";
  for (size_t c = 0; c < P.out.size(); ++c) {
    const int d = 2 * P.out[c].l + 1;
    s << "  {" << P.offo[c] << ", " << d << ", " << P.out[c].mul << ", " << reg << ", " << (usedo[c] ? "true" : "false")
      << "},\n";
    if (usedo[c]) reg += d;
  }
  s << "};\nconstexpr int ACC_REGS = " << reg << ";\n";
  if (reg > 256) return fail(E3X_ERR_INVALID, "uvw kernel: more than 256 output components per multiplicity index");
  NzList L = emit_nz(P, K.path_ids);
  // shared weights of few (u, v) pairs live in registers, one per pair and lane (one chunk of output channels only)
  long long pairs = 0;
  for (const auto& p : P.paths) pairs += (long long)P.in1[p.in1].mul * P.in2[p.in2].mul;
  const bool cached = all_uvw && P.shared_weights && K.chunks == 1 && pairs > 0 && pairs <= 64;
  K.cached_weights = cached;
  s << "constexpr int W_CACHE_REGS = " << (cached ? pairs : 0) << ";\n";
  s << "struct Path { int x1off, d1, U, x2off, d2, V, out, woff, wreg, mode; bool has_w; int nz_beg, nz_end; };\n";
  s << "constexpr int N_PATH = " << P.paths.size() << ";\nconstexpr Path paths[N_PATH > 0 ? N_PATH : 1] = {\n";
  int wreg = 0;
  for (size_t i = 0; i < P.paths.size(); ++i) {
    const auto& p = P.paths[i];
    s << "  {" << P.off1[p.in1] << ", " << 2 * P.in1[p.in1].l + 1 << ", " << P.in1[p.in1].mul << ", " << P.off2[p.in2]
      << ", " << 2 * P.in2[p.in2].l + 1 << ", " << P.in2[p.in2].mul << ", " << p.out << ", " << p.woff << ", " << wreg
      << ", " << p.mode << ", " << (p.has_w ? "true" : "false") << ", " << L.beg[i] << ", " << L.end[i] << "},\n";
    wreg += P.in1[p.in1].mul * P.in2[p.in2].mul;
  }
  if (P.paths.empty()) s << "  {0, 1, 0, 0, 1, 0, 0, 0, 0, 0, false, 0, 0}\n";
  s << "};\n";
  emit_nz_table(s, L);
  s << "}  // namespace cfg\n";
  *src = s.str() + e3x::kTplCommon + e3x::kTplUvwSmall;
  return E3X_OK;
}

// ---- uvw on the matrix cores ----------------------------------------------------------
// largest GEMM K extent (multiplicity of the K operand) of the matrix-core kernels: the fp32 kernel keeps a
// 64-row slice of the K operand in LDS (K * 256 bytes), the bf16 kernel keeps its K operand in registers
int k_cap(int dtype) { return dtype == E3X_BF16 ? 256 : 512; }

bool uvw_mfma_eligible(const e3x_plan& P, int dtype) {
  if (!P.shared_weights || P.paths.empty()) return false;
  for (const auto& p : P.paths) {
    const int U = P.in1[p.in1].mul, V = P.in2[p.in2].mul, W = P.out[p.out].mul;
    // 32-channel granularity (a half-filled last tile)
    if (W % 32 || P.out[p.out].l > 3 || U < 1 || V < 1) return false;
    const int kcap = k_cap(dtype);
    const bool okU = U % 32 == 0 && U <= kcap, okV = V % 32 == 0 && V <= kcap;
    if (dtype == E3X_BF16) {
      // both multiplicities tile: the outer index runs in blocks of 8
      if (!okU || !okV) return false;
      // the bf16 kernel reads 8 consecutive bf16 of a row with one 16-byte load
      if ((P.off1[p.in1] | P.off2[p.in2] | P.in1_dim | P.in2_dim) & 7) return false;
    } else if (!okU && !okV) {
      // fp32: one input's multiplicity is the GEMM K index (multiple of 32), the other's is a plain outer loop of
      // any length -- e.g. node features x a few node attributes, or a linear map (second input "0e")
      return false;
    }
  }
  if (dtype == E3X_BF16) {
    // LDS of the bf16 kernel: four weight buffers of one stage (32 KB each up to 128 K indices, 64 KB above) and two
    // blocks of the R operand for 128 rows
    int kmax = 32, drmax = 1;
    for (const auto& p : P.paths) {
      kmax = std::max(kmax, std::max(P.in1[p.in1].mul, P.in2[p.in2].mul));
      drmax = std::max(drmax, 2 * std::max(P.in1[p.in1].l, P.in2[p.in2].l) + 1);
    }
    const long long stage = (long long)(256 / kmax >= 2 ? 2 : 1) * (kmax / 8) * 64 * 16;
    if (4 * stage + 2LL * drmax * 128 * 16 > 160 * 1024) return false;
  }
  return true;
}
bool uvw_mfma_eligible(const e3x_plan& P) { return uvw_mfma_eligible(P, P.dtype); }

int build_uvw_mfma_source(e3x_plan& P, std::string* src) {
  // Output channels per workgroup.  fp32: 128 (two accumulator tiles per wave, 64 KB of LDS, two workgroups per CU at
  // 256 registers) wherever every output multiplicity is a multiple of 128, else 64 (48 KB, three workgroups at 168
  // registers).  Measured on 128x0e+128x1o+128x2e squared, 65536 rows: 61.3 ms at 64 channels, 56.3 ms at 128 -- a
  // weight chunk then serves twice the matrix work per barrier and per LDS read of the K operand.  The bf16 kernel is
  // written for 64.
  int wt = env_int("E3X_UVW_WT", P.dtype == E3X_F32 ? 128 : 64), kmax = 32;
  for (const auto& p : P.paths)
    if (P.out[p.out].mul % 128) wt = 64;
  if (P.dtype != E3X_F32) wt = 64;
  std::ostringstream s, nzs, ps, ts;
  emit_header(s, P);
  // split-operand matrix steps (see the template) in fp32 storage; weight chunks of 16 K rows then keep the LDS at
  // 72 KB with 128 output channels (two workgroups per CU)
  // Default where every block is a multiple of 64 wide (measured on 128-wide blocks, 65536 rows: 55.9 -> 50.0 ms);
  // narrower blocks leave tiles half empty and keep the fp32 instruction, which needs no splitting.
  bool full = true;
  for (const auto& p : P.paths)
    if (P.in1[p.in1].mul % 64 || P.in2[p.in2].mul % 64 || P.out[p.out].mul % 64) full = false;
  const int split = P.dtype == E3X_F32 ? env_int("E3X_UVW_SPLIT", full ? 1 : 0) : 0;
  if (split) s << "#define E3X_UVW_SPLIT 1\n";
  P.arithmetic = P.dtype != E3X_F32 ? "bf16 matrix instruction" : split ? "bf16 matrix instruction, six products of three-way split operands" : "fp32 matrix instruction";
  if (P.dtype == E3X_F32) s << "#define E3X_UVW_KC " << env_int("E3X_UVW_KC", split ? 16 : 32) << "\n";
  if (env_int("E3X_UVW_KS", 0)) s << "#define E3X_UVW_KS " << env_int("E3X_UVW_KS", 0) << "\n";
  // two waves per SIMD (256 registers) for 128-channel tiles and for l = 3 outputs, whose seven accumulator tiles do not
  // fit the 168 registers of three (64x1o+64x2e squared -> 32x3o: 3122 registers' worth of spills there, none here)
  bool out_l3 = false;
  for (const auto& p : P.paths) out_l3 = out_l3 || P.out[p.out].l >= 3;
  const int wpe = env_int("E3X_UVW_WPE", wt == 128 || out_l3 ? 2 : 0);
  if (wpe) s << "#define E3X_UVW_WPE " << wpe << "\n";
  int n_nz = 0, n_path = 0, n_target = 0, dka = 1, drmax = 1;
  for (size_t c = 0; c < P.out.size(); ++c) {
    std::ostringstream mine;
    const int beg = n_path;
    for (const auto& p : P.paths) {
      if (p.out != (int)c) continue;
      const e3x_irrep &a = P.in1[p.in1], &b = P.in2[p.in2];
      const int d1 = 2 * a.l + 1, d2 = 2 * b.l + 1, d3 = 2 * P.out[c].l + 1;
      // GEMM passes per outer index: 2l+1 of the K operand when accumulators are scaled, 2 l3 + 1 when the
      // operand is synthesised; take the cheapest
      // (the bf16 kernel scales accumulators only: its matrix passes are cheap next to the fp32 epilogue)
      const bool okU = a.mul % 32 == 0 && a.mul <= k_cap(P.dtype), okV = b.mul % 32 == 0 && b.mul <= k_cap(P.dtype);
      const bool synth = P.dtype == E3X_F32 && env_int("E3X_UVW_SYNTH", 1) && d3 < std::min(d1, d2) && okU;
      const bool k_is_x2 = !synth && okV && (!okU || d2 < d1);
      kmax = std::max(kmax, k_is_x2 ? b.mul : a.mul);
      if (synth) dka = std::max(dka, d1);
      drmax = std::max(drmax, k_is_x2 ? d1 : d2);
      const auto& C = e3x::wigner_3j(a.l, b.l, P.out[c].l);
      const int nz_beg = n_nz;
      for (int i = 0; i < d1; ++i)
        for (int j = 0; j < d2; ++j)
          for (int k = 0; k < d3; ++k) {
            const double cv = C[(i * d2 + j) * d3 + k] * p.pw;
            if (cv != 0.0) {
              nzs << "  {" << (k_is_x2 ? j : i) << ", " << (k_is_x2 ? i : j) << ", " << k << ", " << fstr(cv) << "},\n";
              ++n_nz;
            }
          }
      const long long W = P.out[c].mul;
      // W_p[u, v, w] at woff + (u * V + v) * W + w
      const long long stride_u = (long long)b.mul * W, stride_v = W;
      mine << "  {" << (synth ? "true" : "false") << ", " << (k_is_x2 ? "true" : "false") << ", "
           << (k_is_x2 ? P.off2[p.in2] : P.off1[p.in1]) << ", "
           << (k_is_x2 ? d2 : d1) << ", " << (k_is_x2 ? b.mul : a.mul) << ", "
           << (k_is_x2 ? P.off1[p.in1] : P.off2[p.in2]) << ", " << (k_is_x2 ? d1 : d2) << ", "
           << (k_is_x2 ? a.mul : b.mul) << ", " << W << ", " << p.woff << ", " << (k_is_x2 ? stride_v : stride_u) << ", "
           << (k_is_x2 ? stride_u : stride_v) << ", " << nz_beg << ", " << n_nz << "},\n";
      ++n_path;
    }
    if (n_path == beg) continue;
    ps << mine.str();
    for (int w0 = 0; w0 < P.out[c].mul; w0 += wt) {
      ts << "  {" << P.offo[c] << ", " << 2 * P.out[c].l + 1 << ", " << w0 << ", " << std::min(wt, P.out[c].mul - w0) << ", "
         << beg << ", " << n_path << "},\n";
      ++n_target;
    }
  }
  s << "constexpr int WT = " << wt << ", KMAX = " << kmax << ";\n";  // KMAX: the largest GEMM K extent
  for (const char* knob : {"E3X_UVW16_OS", "E3X_UVW16_NBUF", "E3X_UVW16_LEAD", "E3X_UVW16_RT2", "E3X_UVW16_RT2_ROWS", "E3X_UVW16_SHIFT", "E3X_UVW16_SHIFT1"})
    if (P.dtype == E3X_BF16 && std::getenv(knob)) s << "#define " << knob << " " << env_int(knob, 0) << "\n";
  s << "struct Nz { int s, r, k; float c; };\nconstexpr int N_NZ = " << n_nz << ";\nconstexpr Nz nz[N_NZ] = {\n"
    << nzs.str() << "};\n";
  s << "constexpr int DKA = " << dka << ", DRMAX = " << drmax << ";\n";
  s << "struct MPath { bool synth, k_is_x2; int koff, dK, K, roff, dR, O, W; long long wbase, wk_stride, wo_stride; "
       "int nz_beg, nz_end; };\n";
  s << "constexpr int N_MPATH = " << n_path << ";\nconstexpr MPath mpaths[N_MPATH] = {\n" << ps.str() << "};\n";
  s << "struct Target { int out_off, d3, w0, wn, path_beg, path_end; };\n";  // wn: channels in the tile (64, or 32 at the end)
  s << "constexpr int N_TARGET = " << n_target << ";\nconstexpr Target targets[N_TARGET] = {\n" << ts.str() << "};\n";
  s << "}  // namespace cfg\n";
  P.n_targets = n_target;
  *src = s.str() + e3x::kTplCommon + (P.dtype == E3X_BF16 ? e3x::kTplUvwMfmaBf16 : e3x::kTplUvwMfma);
  return E3X_OK;
}

// ---- uvw with a scalar second input (node-wise linear layers) on the matrix cores ------------------
// A target (one output irrep x 32 channels) keeps the weights of all its paths in LDS: at most this many blocks of
// 8 x 32 floats (144 KB, one workgroup per CU; up to 64 KB two or three).  Measured on 128x0e+128x1o+128x2e x S
// species, 50 000 rows, against the kernels these shapes took with a limit of 64 blocks: S = 6 (96 blocks) 0.78 against
// 1.10 ms in fp32 and 0.58 against 2.37 ms in bf16 storage, S = 8 (128 blocks) 1.04 against 1.33 and 0.72 against 2.84 ms.
int node_max_blocks() { return env_int("E3X_NODE_MAX_BLOCKS", 144); }

bool uvw_node_eligible(const e3x_plan& P) {
  if (!P.shared_weights || P.paths.empty() || env_int("E3X_UVW_NODE", 1) == 0) return false;
  if (P.in2_dim < 1 || P.in2_dim > 16 || P.in1_dim % 4) return false;
  for (const auto& r : P.in2) if (r.l != 0) return false;
  std::vector<int> blocks(P.out.size(), 0);
  long long pairs = 0;
  for (const auto& p : P.paths) {
    const e3x_irrep &a = P.in1[p.in1], &b = P.in2[p.in2], &c = P.out[p.out];
    // rows are read in 16-byte pieces of 4 multiplicity indices, 8 indices per matrix-core block
    if (p.mode != E3X_MODE_UVW || a.l != c.l || a.l > 3 || a.mul % 8 || P.off1[p.in1] % 4) return false;
    // the coupling with a scalar is a multiple of the identity
    const auto& C = e3x::wigner_3j(a.l, 0, c.l);
    const int d = 2 * a.l + 1;
    for (int i = 0; i < d; ++i)
      for (int k = 0; k < d; ++k)
        if (std::fabs(C[i * d + k] - (i == k ? C[0] : 0.0)) > 1e-12) return false;
    blocks[p.out] += a.mul / 8 * b.mul;
    pairs += (long long)a.mul * b.mul;
  }
  for (int n : blocks) if (n > node_max_blocks()) return false;
  // a handful of (u, v) pairs in shapes the other matrix-core kernel does not take: the vector-ALU kernel keeps the
  // weights in registers and needs no padding to 32 channels
  // (the same choice in both storages: the tiling rule asked is the fp32 kernel's)
  return pairs > env_int("E3X_NODE_MIN_PAIRS", 64) || uvw_mfma_eligible(P, E3X_F32);
}

int build_uvw_node_source(e3x_plan& P, std::string* src) {
  struct T { int out, w0; long long work; };
  std::vector<T> targets;
  for (size_t c = 0; c < P.out.size(); ++c) {
    long long blocks = 0;
    for (const auto& p : P.paths) if (p.out == (int)c) blocks += P.in1[p.in1].mul / 8 * P.in2[p.in2].mul;
    if (!blocks) continue;
    for (int w0 = 0; w0 < P.out[c].mul; w0 += 32) targets.push_back({(int)c, w0, blocks * (2 * P.out[c].l + 1)});
  }
  // heaviest first: the grid is walked in this order and the light targets fill its tail
  std::stable_sort(targets.begin(), targets.end(), [](const T& a, const T& b) { return a.work > b.work; });
  std::ostringstream s, ps, ts;
  emit_header(s, P);
  int n_path = 0, max_blocks = 1, max_d = 1;
  P.node_tile_rows.clear();
  for (const T& t : targets) {
    const int d = 2 * P.out[t.out].l + 1;
    // rows per wave: 32; 64 for scalars, where one row set would leave a single chain of dependent matrix instructions
    const int rs = env_int("E3X_NODE_RS", d == 1 ? 2 : 1);
    if (rs != 1 && rs != 2) return fail(E3X_ERR_INVALID, "E3X_NODE_RS must be 1 or 2");
    // register sets of the load ring: about twelve 16-byte loads per lane in flight
    const int nbuf = std::max(2, std::min(8, env_int("E3X_NODE_INFLIGHT", 12) / (d * rs)));
    max_d = std::max(max_d, d);
    const int beg = n_path;
    int blocks = 0;
    for (const auto& p : P.paths) {
      if (p.out != t.out) continue;
      const e3x_irrep &a = P.in1[p.in1], &b = P.in2[p.in2];
      const double c = e3x::wigner_3j(a.l, 0, a.l)[0] * p.pw;
      ps << "  {" << P.off1[p.in1] << ", " << a.mul << ", " << P.off2[p.in2] << ", " << b.mul << ", " << p.woff << ", "
         << blocks << ", " << fstr(c) << "},\n";
      blocks += a.mul / 8 * b.mul;
      ++n_path;
    }
    max_blocks = std::max(max_blocks, blocks);
    ts << "  {" << P.offo[t.out] << ", " << d << ", " << t.w0 << ", " << P.out[t.out].mul << ", " << rs << ", " << nbuf << ", "
       << beg << ", " << n_path << "},\n";
    P.node_tile_rows.push_back(128 * rs);
  }
  // W_p[u, v, w] at wbase + (u * O + v) * W + w; lds_block: first LDS block of the path inside its target
  s << "struct NPath { int x_off, U, o_off, O; long long wbase; int lds_block; float c; };\n";
  s << "constexpr int N_NPATH = " << n_path << ";\nconstexpr NPath npaths[N_NPATH] = {\n" << ps.str() << "};\n";
  s << "struct NTarget { int out_off, d, w0, W, rs, nbuf, path_beg, path_end; };\n";
  s << "constexpr int N_NTARGET = " << targets.size() << ";\nconstexpr NTarget ntargets[N_NTARGET] = {\n" << ts.str() << "};\n";
  bool w_aligned = true;  // weight rows of every path are whole 16-byte pieces
  for (const auto& p : P.paths) w_aligned = w_aligned && P.out[p.out].mul % 4 == 0 && p.woff % 4 == 0;
  s << "constexpr bool W_ALIGNED = " << (w_aligned ? "true" : "false") << ";\n";
  s << "constexpr int MAX_BLOCKS = " << max_blocks << ";\n";
  {
    // matrix steps on split operands (see the template) where every input multiplicity is a multiple of 16
    bool split = true;
    for (const auto& p : P.paths) split = split && P.in1[p.in1].mul % 16 == 0;
    split = split && env_int("E3X_NODE_SPLIT", 1) != 0;
    if (split) s << "#define E3X_NODE_SPLIT 1\n";
    P.arithmetic = split ? "bf16 matrix instruction, six products of three-way split operands" : "fp32 matrix instruction";
  }
  // workgroups per CU the register budget is set for: three when their weights fit (160 KB of LDS per CU)
  s << "constexpr int MIN_WGS = " << env_int("E3X_NODE_WGS", max_blocks <= 48 && max_d <= 5 ? 3 : 2) << ";\n";
  s << "}  // namespace cfg\n";
  *src = s.str() + e3x::kTplCommon + e3x::kTplUvwNode;
  return E3X_OK;
}

// The matrix-core weight-gradient kernel reads 8 multiplicity indices of the M operand and of the output gradient
// with 16-byte loads: every irrep offset it starts from and both row lengths must be multiples of 4 floats.  Plans
// that do not fit (an odd total dimension, an irrep of odd size in front of the operand) take the vector-ALU kernel.
bool mfma_dw_fits(const e3x_plan& P) {
  for (const auto& p : P.paths) {
    const e3x_irrep &a = P.in1[p.in1], &b = P.in2[p.in2];
    const bool okU = a.mul % 32 == 0 && a.mul <= k_cap(P.dtype), okV = b.mul % 32 == 0 && b.mul <= k_cap(P.dtype);
    const bool m_is_x2 = okV && (!okU || b.l < a.l);
    const int moff = m_is_x2 ? P.off2[p.in2] : P.off1[p.in1];
    const int64_t mdim = m_is_x2 ? P.in2_dim : P.in1_dim;
    if ((moff | P.offo[p.out] | mdim | P.out_dim) & 3) return false;
  }
  return true;
}

// Tables of the matrix-core weight-gradient kernel: per path the M operand is the input with the smaller l.

int build_uvw_mfma_dw_source(e3x_plan& P, std::string* src) {
  std::ostringstream s, nzs, ps;
  emit_header(s, P);
  if (env_int("E3X_DW_ZC", 0)) s << "#define E3X_DW_ZC " << env_int("E3X_DW_ZC", 0) << "\n";
  if (std::getenv("E3X_DW_SYNTH")) s << "#define E3X_DW_SYNTH " << env_int("E3X_DW_SYNTH", 1) << "\n";
  if (std::getenv("E3X_DW_PAIR")) s << "#define E3X_DW_PAIR " << env_int("E3X_DW_PAIR", 1) << "\n";
  {
    // Split operands (six bf16 products per fp32 one) pay where the 64 x 64 tiles are full: the vector ALU then
    // prepares operands for 4 x 12 matrix instructions per pass; with 32-wide blocks half of them multiply padding and
    // the fp32 instruction, which needs no splitting, is faster (measured: 128-wide blocks 73 -> 60 ms, the 32-wide
    // node-wise layers of the convolution block 0.71 -> 0.78 ms).  A 32-channel path whose outer indices go two to a
    // tile (E3X_DW_PAIR in the template) has no padded columns either: those layers 0.25 -> 0.19 and 0.11 -> 0.09 ms.
    bool full = true;
    const bool pairing = env_int("E3X_DW_PAIR", 1) != 0;
    for (const auto& p : P.paths) {
      const e3x_irrep &a = P.in1[p.in1], &b = P.in2[p.in2], &c = P.out[p.out];
      const int d1 = 2 * a.l + 1, d2 = 2 * b.l + 1;
      const bool okU = a.mul % 32 == 0 && a.mul <= k_cap(P.dtype), okV = b.mul % 32 == 0 && b.mul <= k_cap(P.dtype);
      const bool k_is_x2 = okV && (!okU || d2 < d1);
      const int O = k_is_x2 ? a.mul : b.mul, dK = k_is_x2 ? d2 : d1;
      const bool synth_a = c.l == 0 && dK > 1;
      const bool paired = pairing && c.mul == 32 && O % 2 == 0 && !synth_a;
      if (!paired && ((k_is_x2 ? b.mul : a.mul) % 64 || c.mul % 64)) full = false;
    }
    const int split = env_int("E3X_DW_SPLIT", full ? 1 : 0);
    s << "#define E3X_DW_SPLIT " << split << "\n";
    P.arithmetic_dw = split ? "bf16 matrix instruction, six products of three-way split operands" : "fp32 matrix instruction";
  }
  if (std::getenv("E3X_DW_OCC")) s << "#define E3X_DW_OCC " << env_int("E3X_DW_OCC", 3) << "\n";
  int n_nz = 0, n_path = 0, dkmax = 1, drmax = 1;
  long long tiles = 0;
  if (!mfma_dw_fits(P))
    return fail(E3X_ERR_INVALID, "weight gradient on the matrix cores: irrep offsets and row lengths must be multiples of 4");
  for (const auto& p : P.paths) {
    const e3x_irrep &a = P.in1[p.in1], &b = P.in2[p.in2], &c = P.out[p.out];
    const int d1 = 2 * a.l + 1, d2 = 2 * b.l + 1, d3 = 2 * c.l + 1;
    const bool okU = a.mul % 32 == 0 && a.mul <= k_cap(P.dtype), okV = b.mul % 32 == 0 && b.mul <= k_cap(P.dtype);
    const bool k_is_x2 = okV && (!okU || d2 < d1);  // the M operand tiles by 32
    const auto& C = e3x::wigner_3j(a.l, b.l, c.l);
    const int nz_beg = n_nz;
    for (int i = 0; i < d1; ++i)
      for (int j = 0; j < d2; ++j)
        for (int k = 0; k < d3; ++k) {
          const double cv = C[(i * d2 + j) * d3 + k] * p.pw;
          if (cv != 0.0) {
            nzs << "  {" << (k_is_x2 ? j : i) << ", " << (k_is_x2 ? i : j) << ", " << k << ", " << fstr(cv) << "},\n";
            ++n_nz;
          }
        }
    const long long W = c.mul;
    const long long stride_u = (long long)b.mul * W, stride_v = W;  // W_p[u, v, w] at woff + (u * V + v) * W + w
    const int dK = k_is_x2 ? d2 : d1, dR = k_is_x2 ? d1 : d2;
    const int K = k_is_x2 ? b.mul : a.mul, O = k_is_x2 ? a.mul : b.mul;
    dkmax = std::max(dkmax, dK);
    drmax = std::max(drmax, dR);
    const int ob = O % 4 == 0 ? 4 : (O % 2 == 0 ? 2 : 1);  // outer indices per workgroup
    ps << "  {" << (k_is_x2 ? "true" : "false") << ", " << (k_is_x2 ? P.off2[p.in2] : P.off1[p.in1]) << ", " << dK << ", "
       << K << ", " << (k_is_x2 ? P.off1[p.in1] : P.off2[p.in2]) << ", " << dR << ", " << O << ", " << ob << ", " << P.offo[p.out]
       << ", " << d3 << ", " << W << ", " << p.woff << ", " << (k_is_x2 ? stride_v : stride_u) << ", "
       << (k_is_x2 ? stride_u : stride_v) << ", " << nz_beg << ", " << n_nz << "},\n";
    tiles = std::max(tiles, (long long)((K + 63) / 64) * ((W + 63) / 64) * (O / ob));
    ++n_path;
  }
  s << "constexpr int WT = 64, OBMAX = 4, DKMAX = " << dkmax << ", DRMAX = " << drmax << ";\n";
  s << "struct Nz { int s, r, k; float c; };\nconstexpr int N_NZ = " << n_nz << ";\nconstexpr Nz nz[N_NZ] = {\n"
    << nzs.str() << "};\n";
  s << "struct DPath { bool k_is_x2; int koff, dK, K, roff, dR, O, OB, goff, d3, W; long long wbase, wk_stride, wo_stride; "
       "int nz_beg, nz_end; };\n";
  s << "constexpr int N_DPATH = " << n_path << ";\nconstexpr DPath dpaths[N_DPATH] = {\n" << ps.str() << "};\n";
  s << "}  // namespace cfg\n";
  P.dw_tiles = tiles;
  P.dw_paths = n_path;
  *src = s.str() + e3x::kTplCommon + e3x::kTplUvwMfmaDw;
  return E3X_OK;
}

// builds (or finds in the cache) the weight-gradient code object of a uvw_mfma plan
int prepare_mfma_dw(e3x_plan* P) {
  std::lock_guard<std::mutex> lock(P->mu);
  if (P->dw) return E3X_OK;
  std::unique_ptr<SubKernel> K(new SubKernel);
  std::string src;
  int rc;
  if ((rc = build_uvw_mfma_dw_source(*P, &src))) return rc;
  if ((rc = e3x::get_code_object("uvw_mfma_dw", src, &K->key, &K->hsaco))) return rc;
  P->dw = std::move(K);
  return E3X_OK;
}

int load_dw_function(e3x_plan* P, int dev) {
  std::lock_guard<std::mutex> lock(P->mu);
  SubKernel* K = P->dw.get();
  if (K->module[dev]) return E3X_OK;
  hipModule_t mod = nullptr;
  hipError_t err = hipModuleLoad(&mod, K->hsaco.c_str());
  if (err != hipSuccess) return fail(E3X_ERR_HIP, "hipModuleLoad(" + K->hsaco + ") failed: " + hipGetErrorString(err));
  if (hipModuleGetFunction(&K->fn_dw[dev], mod, "e3x_uvw_mfma_dw") != hipSuccess)
    return fail(E3X_ERR_HIP, "kernel e3x_uvw_mfma_dw missing from " + K->hsaco);
  K->module[dev] = mod;
  return E3X_OK;
}

// A uvw_node or uvw_mfma plan that the matrix-core gradient kernel does not take (multiplicities that are not
// multiples of 32, operands that are not 16-byte aligned within their rows) gets its weight gradient from the
// vector-ALU family: that code object is built on first use.  Decided from the plan alone, so that
// e3x_tp_plan_prepare_backward_w and e3x_tp_backward_w_uvw agree.
bool node_dw_on_valu(const e3x_plan* P) {
  if (P->family == "uvw_node") return !uvw_mfma_eligible(*P) || !mfma_dw_fits(*P);
  if (P->family == "uvw_mfma") return !mfma_dw_fits(*P);
  return false;
}

int prepare_valu_dw(e3x_plan* P) {
  std::lock_guard<std::mutex> lock(P->mu);
  if (P->dw) return E3X_OK;
  std::unique_ptr<SubKernel> K(new SubKernel);
  for (size_t i = 0; i < P->paths.size(); ++i) K->path_ids.push_back((int)i);
  std::string src;
  int rc;
  if ((rc = build_uvw_small_source(*P, *K, &src))) return rc;
  if ((rc = e3x::get_code_object("uvw_small", src, &K->key, &K->hsaco))) return rc;
  P->dw = std::move(K);
  return E3X_OK;
}

int load_valu_dw_function(e3x_plan* P, int dev) {
  std::lock_guard<std::mutex> lock(P->mu);
  SubKernel* K = P->dw.get();
  if (K->module[dev]) return E3X_OK;
  hipModule_t mod = nullptr;
  hipError_t err = hipModuleLoad(&mod, K->hsaco.c_str());
  if (err != hipSuccess) return fail(E3X_ERR_HIP, "hipModuleLoad(" + K->hsaco + ") failed: " + hipGetErrorString(err));
  if (hipModuleGetFunction(&K->fn_dw[dev], mod, "e3x_uvw_small_dw") != hipSuccess)
    return fail(E3X_ERR_HIP, "kernel e3x_uvw_small_dw missing from " + K->hsaco);
  K->module[dev] = mod;
  return E3X_OK;
}

int load_functions(e3x_plan* P, int dev) {
  std::lock_guard<std::mutex> lock(P->mu);
  for (auto& K : P->subs) {
    if (K->module[dev]) continue;
    hipModule_t mod = nullptr;
    hipError_t err = hipModuleLoad(&mod, K->hsaco.c_str());
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, "hipModuleLoad(" + K->hsaco + ") failed: " + hipGetErrorString(err));
    const std::string plain = "e3x_" + P->family + "_plain";
    if (hipModuleGetFunction(&K->fn_plain[dev], mod, plain.c_str()) != hipSuccess)
      return fail(E3X_ERR_HIP, "kernel " + plain + " missing from " + K->hsaco);
    if (P->family == "uvu") {
      if (hipModuleGetFunction(&K->fn_fused[dev], mod, "e3x_uvu_fused") != hipSuccess)
        return fail(E3X_ERR_HIP, "kernel e3x_uvu_fused missing from " + K->hsaco);
    }
    if (P->family == "uvw_mfma" && P->dtype == E3X_BF16) {
      if (hipModuleGetFunction(&K->fn_pack[dev], mod, "e3x_uvw_mfma_pack") != hipSuccess)
        return fail(E3X_ERR_HIP, "kernel e3x_uvw_mfma_pack missing from " + K->hsaco);
    }
    if (P->family == "uvw_small") {
      if (hipModuleGetFunction(&K->fn_dw[dev], mod, "e3x_uvw_small_dw") != hipSuccess)
        return fail(E3X_ERR_HIP, "kernel e3x_uvw_small_dw missing from " + K->hsaco);
    }
    K->module[dev] = mod;
  }
  if (P->msg_mfma && !P->msg_mfma->module[dev]) {
    SubKernel* K = P->msg_mfma.get();
    hipModule_t mod = nullptr;
    hipError_t err = hipModuleLoad(&mod, K->hsaco.c_str());
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, "hipModuleLoad(" + K->hsaco + ") failed: " + hipGetErrorString(err));
    if (hipModuleGetFunction(&K->fn_fused[dev], mod, "e3x_uvu_mfma_fused") != hipSuccess ||
        hipModuleGetFunction(&K->fn_pack[dev], mod, "e3x_uvu_mfma_pack_x1") != hipSuccess)
      return fail(E3X_ERR_HIP, "kernel e3x_uvu_mfma_fused / e3x_uvu_mfma_pack_x1 missing from " + K->hsaco);
    K->module[dev] = mod;
  }
  return E3X_OK;
}

// builds (or finds in the cache) the backward code objects of a uvu plan
int prepare_uvu_bwd(e3x_plan* P) {
  std::lock_guard<std::mutex> lock(P->mu);
  for (auto& K : P->subs) {
    if (K->bwd) continue;
    std::unique_ptr<SubKernel> B(new SubKernel);
    B->path_ids = K->path_ids;
    std::string src;
    int rc;
    if ((rc = build_uvu_source(*P, *B, &src, true))) return rc;
    if ((rc = e3x::get_code_object("uvu_bwd", src, &B->key, &B->hsaco))) return rc;
    K->bwd = std::move(B);
  }
  return E3X_OK;
}

int load_uvu_bwd_functions(e3x_plan* P, int dev) {
  std::lock_guard<std::mutex> lock(P->mu);
  for (auto& K : P->subs) {
    SubKernel* B = K->bwd.get();
    if (B->module[dev]) continue;
    hipModule_t mod = nullptr;
    hipError_t err = hipModuleLoad(&mod, B->hsaco.c_str());
    if (err != hipSuccess) return fail(E3X_ERR_HIP, "hipModuleLoad(" + B->hsaco + ") failed: " + hipGetErrorString(err));
    if (hipModuleGetFunction(&B->fn_bwd_edge[dev], mod, "e3x_uvu_bwd_edge") != hipSuccess)
      return fail(E3X_ERR_HIP, "kernel e3x_uvu_bwd_edge missing from " + B->hsaco);
    if (B->bwd_lds && hipModuleGetFunction(&B->fn_bwd_edge_lds[dev], mod, "e3x_uvu_bwd_edge_lds") != hipSuccess)
      return fail(E3X_ERR_HIP, "kernel e3x_uvu_bwd_edge_lds missing from " + B->hsaco);
    B->module[dev] = mod;
  }
  return E3X_OK;
}

// The fused kernel of a transposed message plan that also writes the per-edge weight gradient: fp32, per-edge
// weights; every kernel of the plan (instruction sets split over disjoint output irreps have several) gets a
// companion, and in each a lane group must own a whole row (one chunk).
bool fused_dw_fits(const e3x_plan* P) {
  if (!(env_int("E3X_UVU_FUSED_DW", 1) != 0 && P->family == "uvu" && P->dtype == E3X_F32 && !P->shared_weights &&
        P->weight_numel > 0 && !P->subs.empty()))
    return false;
  for (const auto& K : P->subs)
    if (K->chunks != 1) return false;
  return true;
}

int prepare_uvu_fused_dw(e3x_plan* P) {
  std::lock_guard<std::mutex> lock(P->mu);
  for (auto& K : P->subs) {
    if (K->fused_dw) continue;
    std::unique_ptr<SubKernel> D(new SubKernel);
    D->path_ids = K->path_ids;
    std::string src;
    const std::string extra = "#define E3X_UVU_FUSED_DW 1\n";
    int rc;
    // (naming the template switches off the row staging and the row reduction through LDS, which this kernel does not use)
    if ((rc = build_uvu_source(*P, *D, &src, false, &extra, e3x::kTplUvu))) return rc;
    if (D->chunks != 1) return fail(E3X_ERR_INVALID, "fused weight gradient: the instruction set needs several chunks");
    if ((rc = e3x::get_code_object("uvu_fdw", src, &D->key, &D->hsaco))) return rc;
    K->fused_dw = std::move(D);
  }
  return E3X_OK;
}

int load_uvu_fused_dw_function(e3x_plan* P, int dev) {
  std::lock_guard<std::mutex> lock(P->mu);
  for (auto& K : P->subs) {
    SubKernel* D = K->fused_dw.get();
    if (D->module[dev]) continue;
    hipModule_t mod = nullptr;
    hipError_t err = hipModuleLoad(&mod, D->hsaco.c_str());
    if (err != hipSuccess) return fail(E3X_ERR_HIP, "hipModuleLoad(" + D->hsaco + ") failed: " + hipGetErrorString(err));
    if (hipModuleGetFunction(&D->fn_fused_dw[dev], mod, "e3x_uvu_fused_dw") != hipSuccess ||
        hipModuleGetFunction(&D->fn_fused_dw_x2[dev], mod, "e3x_uvu_fused_dw_x2") != hipSuccess)
      return fail(E3X_ERR_HIP, "kernel e3x_uvu_fused_dw missing from " + D->hsaco);
    D->module[dev] = mod;
  }
  return E3X_OK;
}

// ---- uvu message kernel with the spherical harmonics formed in the kernel -------------------------------------
// lmax when irreps_in2 is 1x0e + 1x1o + ... + 1x(lmax)(parity (-1)^l) with 1 <= lmax <= 3, else -1
int sh_lmax_of(const e3x_plan* P) {
  const int n = (int)P->in2.size();
  if (P->family != "uvu" || n < 2 || n > 4) return -1;
  for (int l = 0; l < n; ++l)
    if (P->in2[l].mul != 1 || P->in2[l].l != l || P->in2[l].p != (l % 2 ? -1 : 1)) return -1;
  return n - 1;
}

int prepare_uvu_sh(e3x_plan* P, int normalize, int normalization) {
  const int lmax = sh_lmax_of(P);
  if (lmax < 0 || (P->shared_weights && P->weight_numel) || normalization < 0 || normalization > 2) return E3X_ERR_INVALID;
  const int key = (normalize ? 4 : 0) + normalization;
  std::lock_guard<std::mutex> lock(P->mu);
  if (P->sh_subs.count(key)) return E3X_OK;
  std::ostringstream x;
  x << "#define E3X_UVU_SH 1\nconstexpr int SH_LMAX = " << lmax << ";\nconstexpr bool SH_NORMALIZE = " << (normalize ? "true" : "false")
    << ";\nconstexpr float SH_SCALE[4] = {";
  for (int l = 0; l < 4; ++l) {
    const double sc = normalization == E3X_NORM_INTEGRAL ? 1.0 / std::sqrt(4.0 * M_PI) : normalization == E3X_NORM_NORM ? 1.0 / std::sqrt(2.0 * l + 1.0) : 1.0;
    x << fstr(sc) << ", ";
  }
  x << "};\n";
  const std::string extra = x.str();
  std::vector<std::unique_ptr<SubKernel>> built;
  for (auto& K : P->subs) {
    std::unique_ptr<SubKernel> S(new SubKernel);
    S->path_ids = K->path_ids;
    std::string src;
    int rc;
    if ((rc = build_uvu_source(*P, *S, &src, false, &extra))) return rc;
    if ((rc = e3x::get_code_object("uvu_sh", src, &S->key, &S->hsaco))) return rc;
    built.push_back(std::move(S));
  }
  P->sh_subs[key] = std::move(built);
  return E3X_OK;
}

int load_uvu_sh_functions(e3x_plan* P, int key, int dev) {
  std::lock_guard<std::mutex> lock(P->mu);
  for (auto& S : P->sh_subs[key]) {
    if (S->module[dev]) continue;
    hipModule_t mod = nullptr;
    hipError_t err = hipModuleLoad(&mod, S->hsaco.c_str());
    if (err != hipSuccess) return fail(E3X_ERR_HIP, "hipModuleLoad(" + S->hsaco + ") failed: " + hipGetErrorString(err));
    if (hipModuleGetFunction(&S->fn_fused[dev], mod, "e3x_uvu_sh_fused") != hipSuccess)
      return fail(E3X_ERR_HIP, "kernel e3x_uvu_sh_fused missing from " + S->hsaco);
    S->module[dev] = mod;
  }
  return E3X_OK;
}

int current_device(int* dev) {
  if (hipGetDevice(dev) != hipSuccess || *dev < 0 || *dev >= kMaxDevices) return fail(E3X_ERR_HIP, "hipGetDevice failed");
  return E3X_OK;
}

}  // namespace

extern "C" int e3x_tp_plan_create(const e3x_tp_desc* d, e3x_plan** out) {
  if (!d || !out) return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: null argument");
  if (d->n_in1 < 0 || d->n_in2 < 0 || d->n_out < 0 || d->n_ins < 0 || (d->n_in1 && !d->in1) || (d->n_in2 && !d->in2) ||
      (d->n_out && !d->out) || (d->n_ins && !d->ins))
    return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: malformed descriptor");
  if (d->dtype != E3X_F32 && d->dtype != E3X_BF16) return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: unknown dtype");
  std::unique_ptr<e3x_plan> P(new e3x_plan);
  P->shared_weights = d->shared_weights ? 1 : 0;
  P->dtype = d->dtype;
  auto take = [&](const e3x_irrep* src, int n, std::vector<e3x_irrep>& dst, std::vector<int>& off, int64_t& dim) -> int {
    dim = 0;
    for (int i = 0; i < n; ++i) {
      if (src[i].mul < 0 || src[i].l < 0 || src[i].l > 12 || (src[i].p != 1 && src[i].p != -1))
        return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: irrep needs mul >= 0, 0 <= l <= 12, p = +-1");
      dst.push_back(src[i]);
      off.push_back((int)dim);
      dim += dim_of(src[i]);
    }
    return E3X_OK;
  };
  int rc;
  if ((rc = take(d->in1, d->n_in1, P->in1, P->off1, P->in1_dim))) return rc;
  if ((rc = take(d->in2, d->n_in2, P->in2, P->off2, P->in2_dim))) return rc;
  if ((rc = take(d->out, d->n_out, P->out, P->offo, P->out_dim))) return rc;

  int n_uvu = 0, n_uvw = 0, n_other = 0;
  std::vector<char> reached(P->out.size(), 0);
  int64_t woff = 0;
  for (int t = 0; t < d->n_ins; ++t) {
    const e3x_instruction& I = d->ins[t];
    if (I.i_in1 < 0 || I.i_in1 >= d->n_in1 || I.i_in2 < 0 || I.i_in2 >= d->n_in2 || I.i_out < 0 || I.i_out >= d->n_out)
      return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: instruction index out of range");
    const e3x_irrep &a = P->in1[I.i_in1], &b = P->in2[I.i_in2], &c = P->out[I.i_out];
    // selection rules (reference _tensor_product.py:294-295)
    if (a.p * b.p != c.p || c.l < std::abs(a.l - b.l) || c.l > a.l + b.l)
      return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: instruction violates the selection rules");
    if (I.mode < E3X_MODE_UVW || I.mode > E3X_MODE_U_LT_VW)
      return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: unknown connection mode");
    // weight block shapes and multiplicity constraints of the connection modes (reference _tensor_product.py:236-262)
    const int64_t U = a.mul, V = b.mul, W = c.mul;
    int64_t n_w = 0;
    bool shape_ok = true, need_w = false;
    switch (I.mode) {
      case E3X_MODE_UVW: n_w = U * V * W, need_w = true; break;
      case E3X_MODE_UVU: n_w = U * V, shape_ok = U == W; break;
      case E3X_MODE_UVV: n_w = U * V, shape_ok = V == W; break;
      case E3X_MODE_UUW: n_w = U * W, shape_ok = U == V && (I.has_weight || W == 1); break;
      case E3X_MODE_UUU: n_w = U, shape_ok = U == V && V == W; break;
      case E3X_MODE_UVUV: n_w = U * V, shape_ok = W == U * V; break;
      case E3X_MODE_UVU_LT_V: n_w = U * (U - 1) / 2, shape_ok = U == V && W == U * (U - 1) / 2; break;
      default: n_w = U * (U - 1) / 2 * W, shape_ok = U == V, need_w = true; break;
    }
    if (!shape_ok) return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: multiplicities do not fit the connection mode");
    if (need_w && !I.has_weight) return fail(E3X_ERR_INVALID, "uvw and u<vw instructions must have weights");
    const bool empty = a.mul == 0 || b.mul == 0 || c.mul == 0;  // dropped, reference _codegen.py:51
    if (!empty) {
      PathInfo p{I.i_in1, I.i_in2, I.i_out, I.mode, I.has_weight ? 1 : 0, I.path_weight, (int)woff};
      P->paths.push_back(p);
      if (I.mode == E3X_MODE_UVU) ++n_uvu;
      else if (I.mode == E3X_MODE_UVW) ++n_uvw;
      else ++n_other;
      reached[I.i_out] = 1;
    }
    if (I.has_weight && !empty) woff += n_w;
  }
  if (woff >= (1LL << 31)) return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: weight_numel must fit in int32");
  P->weight_numel = woff;
  for (size_t c = 0; c < P->out.size(); ++c)
    if (!reached[c] && dim_of(P->out[c]) > 0) P->zero_fill = true;
  // all-uvu and all-uvw instruction sets have their own kernel families; every other set (the six remaining
  // connection modes, or a mixture) takes the general vector-ALU kernel
  const bool general = n_other > 0 || (n_uvu > 0 && n_uvw > 0);
  if (general && d->dtype != E3X_F32)
    return fail(E3X_ERR_INVALID, "e3x_tp_plan_create: connection modes other than uvu / uvw are fp32 only");

  const char* force_small = std::getenv("E3X_UVW_FORCE_VALU");
  std::vector<std::vector<int>> parts;
  if (n_uvw || general) {
    P->family = (!general && uvw_mfma_eligible(*P) && !(force_small && force_small[0] == '1')) ? "uvw_mfma" : "uvw_small";
    if (!general && uvw_node_eligible(*P) && !(force_small && force_small[0] == '1')) P->family = "uvw_node";
    std::vector<int> all(P->paths.size());
    for (size_t i = 0; i < all.size(); ++i) all[i] = (int)i;
    parts.push_back(all);
  } else {
    P->family = "uvu";
    parts = split_uvu_paths(*P);
  }
  if (P->paths.empty()) parts.clear();  // nothing to contract: every entry point fills the outputs with zeros and returns
  for (auto& ids : parts) {
    std::unique_ptr<SubKernel> K(new SubKernel);
    K->path_ids = ids;
    std::string src;
    if (P->family == "uvw_mfma") {
      rc = build_uvw_mfma_source(*P, &src);
      K->waves_per_block = P->dtype == E3X_BF16 ? 8 : 4;
    }
    else if (P->family == "uvw_node") rc = build_uvw_node_source(*P, &src);
    else if (P->family == "uvw_small") rc = build_uvw_small_source(*P, *K, &src);
    else rc = build_uvu_source(*P, *K, &src);
    if (rc) return rc;
    rc = e3x::get_code_object(P->family, src, &K->key, &K->hsaco);
    if (rc == E3X_ERR_COMPILE && P->family == "uvw_mfma" && P->dtype == E3X_BF16 && !env_int("E3X_NO_JIT", 0)) {
      // The bf16 template hands LDS addresses to its LDS-DMA loads as scalar operands of inline assembly.  Where the
      // compiler keeps such an address in a vector register the assembly does not build: the same source with every
      // address forced through readfirstlane (slower by a few per cent) always does.
      rc = e3x::get_code_object(P->family, "#define E3X_UVW16_SCALAR_ADDR 1\n" + src, &K->key, &K->hsaco);
    }
    if (rc) return rc;
    P->key += (P->key.empty() ? "" : "+") + K->key;
    P->subs.push_back(std::move(K));
  }
  if (P->family == "uvu" && env_int("E3X_UVU_MFMA", 1)) {
    std::unique_ptr<SubKernel> K(new SubKernel);
    std::string src;
    if (build_uvu_msg_mfma_source(*P, *K, &src)) {
      if ((rc = e3x::get_code_object("uvu_mfma", src, &K->key, &K->hsaco))) return rc;
      P->key += "+" + K->key;
      P->msg_mfma = std::move(K);
    }
  }
  *out = P.release();
  return E3X_OK;
}

extern "C" int e3x_tp_plan_destroy(e3x_plan* plan) {
  if (!plan) return E3X_OK;
  // code objects stay loaded: kernels of this plan may still be queued on a stream
  delete plan;
  return E3X_OK;
}

extern "C" int e3x_tp_plan_info(const e3x_plan* plan, int64_t* weight_numel, int64_t* in1_dim, int64_t* in2_dim,
                                int64_t* out_dim, const char** family, const char** cache_key) {
  if (!plan) return fail(E3X_ERR_INVALID, "e3x_tp_plan_info: null plan");
  if (weight_numel) *weight_numel = plan->weight_numel;
  if (in1_dim) *in1_dim = plan->in1_dim;
  if (in2_dim) *in2_dim = plan->in2_dim;
  if (out_dim) *out_dim = plan->out_dim;
  if (family) *family = plan->family.c_str();
  if (cache_key) *cache_key = plan->key.c_str();
  return E3X_OK;
}

extern "C" const char* e3x_tp_plan_arithmetic(const e3x_plan* plan, int which) {
  if (!plan) return "";
  return which == 0 ? plan->arithmetic.c_str() : plan->arithmetic_dw.c_str();
}

static int zero_output(e3x_plan* P, void* out, int64_t rows, hipStream_t st) {
  const size_t bytes = (size_t)rows * P->out_dim * (P->dtype == E3X_BF16 ? 2 : 4);
  if (bytes == 0) return E3X_OK;
  return e3x::fill_zero_bytes(out, bytes, st);
}

static bool needs_packed_weights(const e3x_plan* P) { return P->family == "uvw_mfma" && P->dtype == E3X_BF16; }

extern "C" size_t e3x_tp_forward_workspace_bytes(const e3x_plan* P) {
  return (P && needs_packed_weights(P)) ? (size_t)P->weight_numel * 2 : 0;
}

extern "C" int e3x_tp_forward(e3x_plan* P, const void* x1, const void* x2, const void* w, void* out, int64_t Z,
                              void* stream) {
  return e3x_tp_forward_ws(P, x1, x2, w, out, Z, nullptr, 0, stream);
}

extern "C" int e3x_tp_forward_ws(e3x_plan* P, const void* x1, const void* x2, const void* w, void* out, int64_t Z,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_forward: null plan");
  if (Z < 0) return fail(E3X_ERR_INVALID, "e3x_tp_forward: negative batch");
  if (Z == 0 || P->out_dim == 0) return E3X_OK;
  if (!out || (P->in1_dim && !x1) || (P->in2_dim && !x2) || (P->weight_numel && !w))
    return fail(E3X_ERR_INVALID, "e3x_tp_forward: null pointer");
  hipStream_t st = (hipStream_t)stream;
  int dev, rc;
  if ((rc = current_device(&dev))) return rc;
  if (P->zero_fill || P->paths.empty()) {
    if ((rc = zero_output(P, out, Z, st))) return rc;
    if (P->paths.empty()) return E3X_OK;
  }
  if ((rc = load_functions(P, dev))) return rc;
  long long n_rows = Z;
  if (needs_packed_weights(P)) {
    // the matrix-core kernel reads the weights repacked into octets of consecutive K indices
    if (!workspace || workspace_bytes < (size_t)P->weight_numel * 2)
      return fail(E3X_ERR_INVALID, "e3x_tp_forward: this plan needs e3x_tp_forward_ws with a workspace of "
                                   "e3x_tp_forward_workspace_bytes(plan) bytes");
    if (((uintptr_t)x1 | (uintptr_t)x2 | (uintptr_t)workspace) & 15)
      return fail(E3X_ERR_INVALID, "e3x_tp_forward: x1, x2 and the workspace must be 16-byte aligned");
    void* pargs[] = {(void*)&w, (void*)&workspace};
    hipError_t err = hipModuleLaunchKernel(P->subs[0]->fn_pack[dev], (unsigned)(P->weight_numel / 8 / 256), 1, 1, 256, 1, 1,
                                           0, st, pargs, nullptr);
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, std::string("e3x_tp_forward: launch failed: ") + hipGetErrorString(err));
    w = workspace;
  }
  void* args[] = {(void*)&x1, (void*)&x2, (void*)&w, (void*)&out, (void*)&n_rows};
  for (auto& K : P->subs) {
    long long blocks;
    unsigned grid_y = 1;
    if (P->family == "uvw_mfma") {
      const int rows = 16 * K->waves_per_block;  // fp32: 4 waves, 64 rows; bf16: 8 waves, 128 rows
      blocks = (Z + rows - 1) / rows;
      grid_y = (unsigned)P->n_targets;
      // weights that fit in one L2 with room to spare: order the workgroups by row tile (fp32 kernel)
      if (P->dtype == E3X_F32 && P->n_targets > 1 && P->weight_numel * 4 <= (1 << 20) &&
          blocks * P->n_targets < (1LL << 31)) {
        blocks = (blocks + 7) / 8 * 8 * P->n_targets;  // row tiles padded to the 8 XCDs
        grid_y = 1;
      }
    } else if (P->family == "uvw_node") {
      if (((uintptr_t)x1 | (uintptr_t)w) & 15)
        return fail(E3X_ERR_INVALID, "e3x_tp_forward: x1 and the weights must be 16-byte aligned");
      blocks = 0;
      for (int rows : P->node_tile_rows) blocks += (Z + rows - 1) / rows;
    } else {
      const int groups = 64 / K->lanes;
      const long long items = (Z + groups - 1) / groups * K->chunks;
      blocks = (items + K->waves_per_block - 1) / K->waves_per_block;
      if (K->cached_weights) blocks = std::min(blocks, 256LL * 16);  // a few workgroups per CU, each walking many rows
    }
    if (blocks >= (1LL << 31)) return fail(E3X_ERR_INVALID, "e3x_tp_forward: batch too large for one launch");
    hipError_t err =
        hipModuleLaunchKernel(K->fn_plain[dev], (unsigned)blocks, grid_y, 1, 64 * K->waves_per_block, 1, 1, 0, st, args, nullptr);
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, std::string("e3x_tp_forward: launch failed: ") + hipGetErrorString(err));
  }
  return E3X_OK;
}

constexpr int kSrcInRowOrderHost = 2;  // index mode of the kernels: the source ids as an int32 list in sorted position order

// one launch of e3x_uvu_fused per kernel of the set (several when the instruction set is split over output irreps)
static int launch_fused_kernels(const std::vector<std::unique_ptr<SubKernel>>& kernels, int dev, long long n_rows, void** args,
                                hipStream_t st) {
  for (auto& K : kernels) {
    const long long items = n_rows * K->chunks;
    long long blocks = (items + K->waves_per_block - 1) / K->waves_per_block;
    blocks = (blocks + 7) / 8 * 8;  // the kernel deals contiguous eighths of the rows to the 8 XCDs
    if (blocks >= (1LL << 31)) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter: too many rows for one launch");
    hipError_t err = hipModuleLaunchKernel(K->fn_fused[dev], (unsigned)blocks, 1, 1, 64 * K->waves_per_block, 1, 1,
                                           0, st, args, nullptr);
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, std::string("e3x_tp_gather_scatter: launch failed: ") + hipGetErrorString(err));
  }
  return E3X_OK;
}

extern "C" int e3x_tp_gather_scatter(e3x_plan* P, const void* node_x, const void* edge_attr, const void* w,
                                     const void* src, int idx_bits, const int32_t* rowptr, const int32_t* perm,
                                     void* out, int64_t E, int64_t num_src_nodes, int64_t num_out_nodes,
                                     void* stream) {
  return e3x_tp_gather_scatter_ordered(P, node_x, edge_attr, w, src, idx_bits, rowptr, perm, nullptr, out, E,
                                       num_src_nodes, num_out_nodes, stream);
}

extern "C" int e3x_tp_gather_scatter_ordered(e3x_plan* P, const void* node_x, const void* edge_attr, const void* w,
                                             const void* src, int idx_bits, const int32_t* rowptr, const int32_t* perm,
                                             const int32_t* row_order, void* out, int64_t E, int64_t num_src_nodes,
                                             int64_t num_out_nodes, void* stream) {
  return e3x_tp_gather_scatter_ws(P, node_x, edge_attr, w, src, idx_bits, rowptr, perm, row_order, nullptr, out, E,
                                  num_src_nodes, num_out_nodes, nullptr, 0, stream);
}

extern "C" size_t e3x_tp_gather_scatter_workspace_bytes(const e3x_plan* P, int64_t num_src_nodes) {
  if (!P || !P->msg_mfma || num_src_nodes <= 0) return 0;
  return (size_t)num_src_nodes * 128 * 32;  // the node table in operand order: 16 bf16 per multiplicity index
}

extern "C" int e3x_tp_gather_scatter_ws(e3x_plan* P, const void* node_x, const void* edge_attr, const void* w,
                                        const void* src, int idx_bits, const int32_t* rowptr, const int32_t* perm,
                                        const int32_t* row_order, const int32_t* src_rows, void* out, int64_t E,
                                        int64_t num_src_nodes, int64_t num_out_nodes, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter: null plan");
  if (P->family != "uvu") return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter: the plan must be all-uvu");
  if (P->shared_weights && P->weight_numel)
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter: per-edge weights (shared_weights = 0) are required");
  if (idx_bits != 32 && idx_bits != 64) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter: idx_bits must be 32 or 64");
  if (E < 0 || num_src_nodes < 0 || num_out_nodes < 0) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter: negative size");
  if (num_out_nodes == 0 || P->out_dim == 0) return E3X_OK;
  if (!out || !rowptr || (E > 0 && (!src || (P->in1_dim && !node_x) || (P->in2_dim && !edge_attr) || (P->weight_numel && !w))))
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter: null pointer");
  hipStream_t st = (hipStream_t)stream;
  int dev, rc;
  if ((rc = current_device(&dev))) return rc;
  if (P->zero_fill || P->paths.empty()) {
    if ((rc = zero_output(P, out, num_out_nodes, st))) return rc;
    if (P->paths.empty()) return E3X_OK;
  }
  if ((rc = load_functions(P, dev))) return rc;
  // index mode of the kernels: 0 / 1 = the caller's int32 / int64 list indexed by edge id, 2 = src_rows
  int idx64 = idx_bits == 64;
  if (src_rows) {
    src = src_rows;
    idx64 = kSrcInRowOrderHost;
  }
  long long n_rows = num_out_nodes, n_src = num_src_nodes;
  void* args[] = {(void*)&node_x, (void*)&edge_attr, (void*)&w,         (void*)&out,    (void*)&src,  (void*)&idx64,
                  (void*)&rowptr, (void*)&perm,      (void*)&row_order, (void*)&n_rows, (void*)&n_src};
  // the matrix-core message kernel: needs the workspace for the node table in operand order, and 16-byte aligned
  // node table, weights, edge attributes, output and workspace (their rows are whole 16-byte pieces by construction of
  // the kernel, and it reads and writes them as such); without them the vector-ALU kernels below run
  if (P->msg_mfma && E > 0 && workspace && workspace_bytes >= e3x_tp_gather_scatter_workspace_bytes(P, num_src_nodes) &&
      !(((uintptr_t)w | (uintptr_t)edge_attr | (uintptr_t)node_x | (uintptr_t)out | (uintptr_t)workspace) & 15)) {
    SubKernel* K = P->msg_mfma.get();
    {
      const long long pblocks = n_src;  // a workgroup per node
      void* pargs[] = {(void*)&node_x, (void*)&workspace, (void*)&n_src};
      hipError_t perr = hipModuleLaunchKernel(K->fn_pack[dev], (unsigned)pblocks, 1, 1, 256, 1, 1, 0, st, pargs, nullptr);
      if (perr != hipSuccess)
        return fail(E3X_ERR_HIP, std::string("e3x_tp_gather_scatter: launch failed: ") + hipGetErrorString(perr));
    }
    void* margs[] = {(void*)&workspace, (void*)&edge_attr, (void*)&w,         (void*)&out,    (void*)&src,  (void*)&idx64,
                     (void*)&rowptr,    (void*)&perm,      (void*)&row_order, (void*)&n_rows, (void*)&n_src};
    const long long items = n_rows * P->msg_groups;
    long long blocks = (items + K->waves_per_block - 1) / K->waves_per_block;
    blocks = (blocks + 7) / 8 * 8;
    if (blocks >= (1LL << 31)) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter: too many rows for one launch");
    hipError_t err = hipModuleLaunchKernel(K->fn_fused[dev], (unsigned)blocks, 1, 1, 64 * K->waves_per_block, 1, 1, 0,
                                           st, margs, nullptr);
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, std::string("e3x_tp_gather_scatter: launch failed: ") + hipGetErrorString(err));
    return E3X_OK;
  }
  return launch_fused_kernels(P->subs, dev, n_rows, args, st);
}

extern "C" int e3x_tp_plan_prepare_gather_scatter_sh(e3x_plan* P, int32_t normalize, int32_t normalization) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_plan_prepare_gather_scatter_sh: null plan");
  return prepare_uvu_sh(P, normalize, normalization);  // E3X_ERR_INVALID without a message: callers ask to find out
}

extern "C" int e3x_tp_gather_scatter_sh(e3x_plan* P, const void* node_x, const float* edge_vec, const void* w,
                                        const void* src, int idx_bits, const int32_t* rowptr, const int32_t* perm,
                                        const int32_t* row_order, const int32_t* src_rows, void* out, int64_t E,
                                        int64_t num_src_nodes, int64_t num_out_nodes, int32_t normalize,
                                        int32_t normalization, void* stream) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_sh: null plan");
  int rc = prepare_uvu_sh(P, normalize, normalization);
  if (rc == E3X_ERR_INVALID)
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_sh: needs an all-uvu plan with per-edge weights whose second input is 0e + 1o + ... up to l <= 3");
  if (rc) return rc;
  if (idx_bits != 32 && idx_bits != 64) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_sh: idx_bits must be 32 or 64");
  if (E < 0 || num_src_nodes < 0 || num_out_nodes < 0) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_sh: negative size");
  if (num_out_nodes == 0 || P->out_dim == 0) return E3X_OK;
  if (!out || !rowptr || (E > 0 && (!src || (P->in1_dim && !node_x) || !edge_vec || (P->weight_numel && !w))))
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_sh: null pointer");
  hipStream_t st = (hipStream_t)stream;
  int dev;
  if ((rc = current_device(&dev))) return rc;
  if (P->zero_fill || P->paths.empty()) {
    if ((rc = zero_output(P, out, num_out_nodes, st))) return rc;
    if (P->paths.empty()) return E3X_OK;
  }
  const int key = (normalize ? 4 : 0) + normalization;
  if ((rc = load_uvu_sh_functions(P, key, dev))) return rc;
  int idx64 = idx_bits == 64;
  if (src_rows) {
    src = src_rows;
    idx64 = kSrcInRowOrderHost;
  }
  long long n_rows = num_out_nodes, n_src = num_src_nodes;
  void* args[] = {(void*)&node_x, (void*)&edge_vec, (void*)&w,         (void*)&out,    (void*)&src,  (void*)&idx64,
                  (void*)&rowptr, (void*)&perm,     (void*)&row_order, (void*)&n_rows, (void*)&n_src};
  return launch_fused_kernels(P->sh_subs[key], dev, n_rows, args, st);
}

extern "C" int e3x_tp_plan_prepare_gather_scatter_grad_w(e3x_plan* P) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_plan_prepare_gather_scatter_grad_w: null plan");
  if (!fused_dw_fits(P)) return E3X_ERR_INVALID;  // (no message: callers ask to find out)
  return prepare_uvu_fused_dw(P);
}

extern "C" int e3x_tp_gather_scatter_grad_w(e3x_plan* P, const void* table, const void* edge_attr, const void* w,
                                            const void* row_x, const void* gather_idx, int idx_bits,
                                            const int32_t* rowptr, const int32_t* perm, const int32_t* row_order,
                                            const int32_t* src_rows, void* out, void* grad_w, void* grad_x2,
                                            int64_t E, int64_t num_table_rows, int64_t num_out_rows, void* stream) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_grad_w: null plan");
  if (!fused_dw_fits(P))
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_grad_w: needs an all-uvu fp32 plan with per-edge weights whose kernels each cover a row with one chunk");
  if (idx_bits != 32 && idx_bits != 64) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_grad_w: idx_bits must be 32 or 64");
  if (E < 0 || num_table_rows < 0 || num_out_rows < 0) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_grad_w: negative size");
  if (num_out_rows == 0) return E3X_OK;
  if (!out || !rowptr || !row_x || (E > 0 && (!gather_idx || !table || (P->in2_dim && !edge_attr) || !w || !grad_w)))
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_grad_w: null pointer");
  if (((uintptr_t)grad_w) & 15) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_grad_w: grad_w must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  int dev, rc;
  if ((rc = current_device(&dev))) return rc;
  if ((rc = prepare_uvu_fused_dw(P))) return rc;
  if ((rc = load_uvu_fused_dw_function(P, dev))) return rc;
  if (P->zero_fill && (rc = zero_output(P, out, num_out_rows, st))) return rc;
  // index mode of the kernel: 0 / 1 = the caller's int32 / int64 list indexed by edge id, 2 = src_rows
  int idx64 = idx_bits == 64;
  if (src_rows) {
    gather_idx = src_rows;
    idx64 = 2;
  }
  long long n_rows = num_out_rows, n_src = num_table_rows;
  int x2_accumulate = 0;  // the first kernel writes the edge-attribute gradient, the others add their paths' share
  void* args[] = {(void*)&table,  (void*)&edge_attr, (void*)&w,         (void*)&out,    (void*)&gather_idx, (void*)&idx64,
                  (void*)&rowptr, (void*)&perm,      (void*)&row_order, (void*)&n_rows, (void*)&n_src,      (void*)&row_x,
                  (void*)&grad_w, (void*)&grad_x2,   (void*)&x2_accumulate};
  for (auto& K : P->subs) {
    SubKernel* D = K->fused_dw.get();
    long long blocks = (n_rows + D->waves_per_block - 1) / D->waves_per_block;
    blocks = (blocks + 7) / 8 * 8;  // the kernel deals contiguous eighths of the rows to the 8 XCDs
    if (blocks >= (1LL << 31)) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_grad_w: too many rows for one launch");
    hipError_t err = hipModuleLaunchKernel(grad_x2 ? D->fn_fused_dw_x2[dev] : D->fn_fused_dw[dev], (unsigned)blocks, 1, 1,
                                           64 * D->waves_per_block, 1, 1, 0, st, args, nullptr);
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, std::string("e3x_tp_gather_scatter_grad_w: launch failed: ") + hipGetErrorString(err));
    x2_accumulate = 1;
  }
  return E3X_OK;
}

// ---- message step with the radial network inside ---------------------------------------------------------
namespace {

// what the fused kernel assumes about the instruction set
const char* radial_unsupported(const e3x_plan* P) {
  if (P->family != "uvu") return "the plan must be all-uvu";
  if (P->dtype != E3X_F32) return "fp32 storage only";
  if (P->shared_weights || P->paths.empty()) return "per-edge weights are required";
  if (P->in2_dim > 64) return "irreps_in2.dim > 64";
  for (size_t i = 0; i < P->paths.size(); ++i) {
    const PathInfo& p = P->paths[i];
    if (!p.has_w || P->in2[p.in2].mul != 1 || P->in1[p.in1].mul != 32 || P->out[p.out].mul != 32 || p.woff != 32 * (int)i)
      return "every instruction needs a weight, multiplicity 32 on the first input and the output, 1 on the second";
  }
  return nullptr;
}

int prepare_radial(e3x_plan* P, int n_in, int n_hidden, int act, double c1, double c2) {
  std::ostringstream d;
  d << n_in << "/" << n_hidden << "/" << act << "/" << fstr(c1) << "/" << fstr(c2);
  std::lock_guard<std::mutex> lock(P->mu);
  if (!P->radial.empty() && P->radial_desc == d.str()) return E3X_OK;
  std::ostringstream x;
  x << "constexpr int FC_H0 = " << n_in << ", FC_H1 = " << n_hidden << ", FC_ACT = " << act << ";\n";
  x << "constexpr float FC_C1 = " << fstr(c1) << ", FC_C2 = " << fstr(c2) << ";\n";
  if (std::getenv("E3X_UVUFC_SPLIT")) x << "#define E3X_UVUFC_SPLIT " << env_int("E3X_UVUFC_SPLIT", 1) << "\n";
  const std::string extra = x.str();
  // A lane keeps the accumulators of two multiplicity indices next to 8 registers of weights per instruction: above
  // 18 output components per index the instructions are dealt to several kernels over disjoint output irreps (one
  // per group of first-input irreps, so each kernel gathers only its own slice of the source row).
  std::vector<std::unique_ptr<SubKernel>> parts;
  const int acc_limit = env_int("E3X_UVUFC_ACC_LIMIT", 24);
  std::vector<std::vector<int>> groups = split_uvu_paths(*P, acc_limit);
  // neighbouring groups are put together again while their output components stay within the limit
  auto acc_of = [&](const std::vector<int>& ids) {
    std::vector<char> seen(P->out.size(), 0);
    int n = 0;
    for (int id : ids)
      if (!seen[P->paths[id].out]) { seen[P->paths[id].out] = 1; n += 2 * P->out[P->paths[id].out].l + 1; }
    return n;
  };
  for (size_t g = 0; g + 1 < groups.size();) {
    std::vector<int> both = groups[g];
    both.insert(both.end(), groups[g + 1].begin(), groups[g + 1].end());
    if (acc_of(both) <= acc_limit) {
      std::sort(both.begin(), both.end());
      groups[g] = both;
      groups.erase(groups.begin() + g + 1);
    } else {
      ++g;
    }
  }
  for (auto& ids : groups) {
    std::unique_ptr<SubKernel> K(new SubKernel);
    K->path_ids = ids;
    std::string src;
    int rc;
    if ((rc = build_uvu_source(*P, *K, &src, false, &extra, e3x::kTplUvuFc))) return rc;
    if ((rc = e3x::get_code_object("uvu_fc", src, &K->key, &K->hsaco))) return rc;
    parts.push_back(std::move(K));
  }
  for (auto& old : P->radial) P->radial_retired.push_back(std::move(old));
  P->radial = std::move(parts);
  P->radial_desc = d.str();
  return E3X_OK;
}

int load_radial_function(e3x_plan* P, int dev) {
  std::lock_guard<std::mutex> lock(P->mu);
  for (auto& K : P->radial) {
    if (K->module[dev]) continue;
    hipModule_t mod = nullptr;
    hipError_t err = hipModuleLoad(&mod, K->hsaco.c_str());
    if (err != hipSuccess) return fail(E3X_ERR_HIP, "hipModuleLoad(" + K->hsaco + ") failed: " + hipGetErrorString(err));
    if (hipModuleGetFunction(&K->fn_fused[dev], mod, "e3x_uvu_fc_fused") != hipSuccess)
      return fail(E3X_ERR_HIP, "kernel e3x_uvu_fc_fused missing from " + K->hsaco);
    K->module[dev] = mod;
  }
  return E3X_OK;
}

}  // namespace

// validation of the network description and construction of the kernel (shared by the two entry points below)
static int radial_kernel(e3x_plan* P, int32_t n_in, int32_t n_hidden, int32_t act, double act_cst, double variance_in,
                         double variance_out) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_radial: null plan");
  if (const char* why = radial_unsupported(P))
    return fail(E3X_ERR_INVALID, std::string("e3x_tp_gather_scatter_radial: ") + why);
  if (n_in < 1 || n_in > 64 || n_hidden < 16 || n_hidden > 128 || n_hidden % 16)
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_radial: 1..64 inputs and 16..128 hidden units in multiples of 16");
  // the second layer is held as three bf16 planes (6 bytes per weight) when the hidden width is a multiple of 32
  const int64_t packed = (int64_t)((n_in + 3) / 4) * 64 * (n_hidden / 16) * 4 +
                         (int64_t)n_hidden * P->weight_numel * (n_hidden % 32 == 0 ? 6 : 4);
  if (packed > 160 * 1024)
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_radial: the network does not fit the LDS of a compute unit");
  if (act < E3X_ACT_IDENTITY || act > E3X_ACT_RELU) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_radial: unknown activation");
  if (!(variance_in > 0) || !(variance_out > 0)) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_radial: variances must be positive");
  // e3nn/nn/_fc.py:38-48,70-88 for two layers: act(x @ W1 / sqrt(h0 var_in)) * cst @ W2 / sqrt(h1 / var_out)
  const bool has_act = act != E3X_ACT_IDENTITY;
  const double c1 = 1.0 / std::sqrt((double)n_in * variance_in);
  const double c2 = (has_act ? act_cst : 1.0) * std::sqrt(variance_out / (double)n_hidden);
  return prepare_radial(P, n_in, n_hidden, act, c1, c2);
}

extern "C" int e3x_tp_plan_prepare_radial(e3x_plan* P, int32_t n_in, int32_t n_hidden, int32_t act, double act_cst,
                                          double variance_in, double variance_out) {
  return radial_kernel(P, n_in, n_hidden, act, act_cst, variance_in, variance_out);
}

extern "C" int e3x_tp_gather_scatter_radial(e3x_plan* P, const void* node_x, const void* edge_attr,
                                            const void* edge_scalars, const void* w1, const void* w2, int32_t n_in,
                                            int32_t n_hidden, int32_t act, double act_cst, double variance_in,
                                            double variance_out, const void* src, int idx_bits, const int32_t* rowptr,
                                            const int32_t* perm, void* out, int64_t E, int64_t num_src_nodes,
                                            int64_t num_out_nodes, void* stream) {
  int rc;
  if ((rc = radial_kernel(P, n_in, n_hidden, act, act_cst, variance_in, variance_out))) return rc;
  if (idx_bits != 32 && idx_bits != 64) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_radial: idx_bits must be 32 or 64");
  if (E < 0 || num_src_nodes < 0 || num_out_nodes < 0) return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_radial: negative size");
  if (E >= (1LL << 31) || num_src_nodes >= (1LL << 31))
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_radial: edge and node counts must fit in int32");
  if (num_out_nodes == 0 || P->out_dim == 0) return E3X_OK;
  if (!out || !rowptr || (E > 0 && (!src || !node_x || (P->in2_dim && !edge_attr) || !edge_scalars || !w1 || !w2)))
    return fail(E3X_ERR_INVALID, "e3x_tp_gather_scatter_radial: null pointer");
  hipStream_t st = (hipStream_t)stream;
  int dev;
  if ((rc = current_device(&dev))) return rc;
  // rows are written by stores or by atomic additions, rows without edges by nobody: everything starts at zero
  if ((rc = zero_output(P, out, num_out_nodes, st))) return rc;
  if (E == 0) return E3X_OK;
  if ((rc = load_radial_function(P, dev))) return rc;
  int n_cu = 0;
  if (hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n_cu <= 0) n_cu = 256;
  // one persistent workgroup of 8 waves per compute unit, 32 workers (quads) each; no more workers than groups of 4 edges
  long long blocks = std::min<long long>(n_cu, (E + 127) / 128);
  int idx64 = idx_bits == 64;
  long long n_rows = num_out_nodes, n_src = num_src_nodes, n_edges = E;
  void* args[] = {(void*)&node_x, (void*)&edge_attr, (void*)&edge_scalars, (void*)&w1,     (void*)&w2,
                  (void*)&out,    (void*)&src,       (void*)&idx64,        (void*)&rowptr, (void*)&perm,
                  (void*)&n_rows, (void*)&n_src,     (void*)&n_edges};
  std::vector<SubKernel*> parts;
  {
    std::lock_guard<std::mutex> lock(P->mu);
    for (auto& K : P->radial) parts.push_back(K.get());
  }
  for (SubKernel* K : parts) {
    hipError_t err = hipModuleLaunchKernel(K->fn_fused[dev], (unsigned)blocks, 1, 1, 512, 1, 1, 0, st, args, nullptr);
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, std::string("e3x_tp_gather_scatter_radial: launch failed: ") + hipGetErrorString(err));
  }
  return E3X_OK;
}

extern "C" int e3x_tp_backward_w_x2(e3x_plan* P, const void* x1, const void* x2, const void* w, const void* grad_out,
                                    const void* src, const void* dst, int idx_bits, void* grad_w, void* grad_x2,
                                    int64_t E, int64_t num_src_nodes, int64_t num_out_nodes, void* stream) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_x2: null plan");
  if (P->family != "uvu") return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_x2: the plan must be all-uvu");
  if (P->shared_weights && P->weight_numel && grad_w && P->dtype != E3X_F32)
    return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_x2: the gradient of shared weights is fp32 only");
  if (idx_bits != 32 && idx_bits != 64) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_x2: idx_bits must be 32 or 64");
  if (E < 0 || num_src_nodes < 0 || num_out_nodes < 0) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_x2: negative size");
  if ((src == nullptr) != (dst == nullptr))
    return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_x2: give both index arrays or neither");
  if (E == 0 || (!grad_w && !grad_x2)) return E3X_OK;
  // x2 is read by the weight gradient only, per-sample weights by the gradient of the second input only
  if (!grad_out || (P->in1_dim && !x1) || (P->in2_dim && !x2 && grad_w) ||
      (P->weight_numel && !w && (grad_x2 || P->shared_weights)))
    return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_x2: null pointer");
  hipStream_t st = (hipStream_t)stream;
  int dev, rc;
  if ((rc = current_device(&dev))) return rc;
  const size_t esz = P->dtype == E3X_BF16 ? 2 : 4;
  if (P->paths.empty() || P->in2_dim == 0) grad_x2 = P->paths.empty() ? grad_x2 : nullptr;
  if (P->paths.empty()) {
    if (grad_x2 && (rc = e3x::fill_zero_bytes(grad_x2, (size_t)E * P->in2_dim * esz, st))) return rc;
    return E3X_OK;
  }
  if ((rc = prepare_uvu_bwd(P))) return rc;
  if ((rc = load_uvu_bwd_functions(P, dev))) return rc;
  int x2_atomic = 0;
  for (auto& K : P->subs)
    if (K->bwd->chunks > 1) x2_atomic = 1;
  if (P->subs.size() > 1) x2_atomic = 1;
  if (grad_x2 && x2_atomic) {
    if (P->dtype != E3X_F32)
      return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_x2: grad_x2 in bf16 storage needs a single-kernel plan");
    if ((rc = e3x::fill_zero_bytes(grad_x2, (size_t)E * P->in2_dim * esz, st))) return rc;
  }
  // Per-sample weights: every weighted path belongs to exactly one kernel of the plan and every multiplicity index
  // to exactly one lane, so each element of grad_w[E, weight_numel] is stored exactly once -- no zero fill (it would
  // be a second pass over the largest tensor of the call).  Shared weights are accumulated with atomics from zero.
  if (grad_w && P->weight_numel && P->shared_weights &&
      (rc = e3x::fill_zero_bytes(grad_w, (size_t)P->weight_numel * esz, st)))
    return rc;
  int idx64 = idx_bits == 64;
  long long n_edges = E, n_src = num_src_nodes;
  void* args[] = {(void*)&x1,  (void*)&x2,     (void*)&w,       (void*)&grad_out,  (void*)&src,     (void*)&dst,
                  (void*)&idx64, (void*)&grad_w, (void*)&grad_x2, (void*)&x2_atomic, (void*)&n_edges, (void*)&n_src};
  for (auto& F : P->subs) {
    SubKernel* K = F->bwd.get();
    const int groups = 64 / K->lanes;
    const long long items = (E + groups - 1) / groups * K->chunks;
    const long long blocks = (items + K->waves_per_block - 1) / K->waves_per_block;
    if (blocks >= (1LL << 31)) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_x2: too many edges for one launch");
    // rows in 16-byte pieces need aligned rows (their lengths are multiples of four by construction of the variant)
    const bool staged = K->bwd_lds && grad_w && w && x2 && !(((uintptr_t)x1 | (uintptr_t)w | (uintptr_t)grad_out | (uintptr_t)grad_w) & 15);
    hipError_t err = hipModuleLaunchKernel(staged ? K->fn_bwd_edge_lds[dev] : K->fn_bwd_edge[dev], (unsigned)blocks, 1, 1,
                                           64 * K->waves_per_block, 1, 1, 0, st, args, nullptr);
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, std::string("e3x_tp_backward_w_x2: launch failed: ") + hipGetErrorString(err));
  }
  return E3X_OK;
}

extern "C" int e3x_tp_plan_prepare_backward_w(e3x_plan* P) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_plan_prepare_backward_w: null plan");
  if (P->family == "uvw_small")
    for (const auto& q : P->paths)
      if (q.mode != E3X_MODE_UVW)
        return fail(E3X_ERR_INVALID, "e3x_tp_plan_prepare_backward_w: no weight-gradient kernel for connection modes other than uvu / uvw");
  if (node_dw_on_valu(P)) return prepare_valu_dw(P);
  if (P->family == "uvw_mfma" || P->family == "uvw_node") {
    if (P->dtype != E3X_F32) return fail(E3X_ERR_INVALID, "e3x_tp_plan_prepare_backward_w: fp32 storage only");
    return prepare_mfma_dw(P);
  }
  if (P->family == "uvu") return P->paths.empty() ? E3X_OK : prepare_uvu_bwd(P);
  return E3X_OK;  // uvw_small carries its gradient kernel in the forward code object
}

extern "C" int e3x_tp_backward_w_uvw(e3x_plan* P, const void* x1, const void* x2, const void* grad_out, void* grad_w,
                                     int64_t Z, void* stream) {
  if (!P) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_uvw: null plan");
  if (P->family != "uvw_small" && P->family != "uvw_mfma" && P->family != "uvw_node")
    return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_uvw: the plan must be all-uvw");
  // the general vector-ALU family also holds the other connection modes, whose weight blocks are not [U, V, W]
  for (const auto& q : P->paths)
    if (q.mode != E3X_MODE_UVW) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_uvw: the plan must be all-uvw");
  if (P->dtype != E3X_F32) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_uvw: fp32 storage only");
  if (Z < 0) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_uvw: negative batch");
  if (P->weight_numel == 0) return E3X_OK;
  if (!grad_w) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_uvw: null pointer");
  hipStream_t st = (hipStream_t)stream;
  int dev, rc;
  if ((rc = current_device(&dev))) return rc;
  // the node-wise family has no gradient kernel of its own: the matrix-core one where its tiling fits, else the vector-ALU one
  const bool mfma = (P->family == "uvw_mfma" || P->family == "uvw_node") && !node_dw_on_valu(P);
  if (Z == 0) return P->shared_weights ? e3x::fill_zero_bytes(grad_w, (size_t)P->weight_numel * 4, st) : E3X_OK;
  if (!grad_out || (P->in1_dim && !x1) || (P->in2_dim && !x2)) return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_uvw: null pointer");
  long long n_rows = Z;
  if (mfma) {
    if (((uintptr_t)x1 | (uintptr_t)x2 | (uintptr_t)grad_out) & 15)
      return fail(E3X_ERR_INVALID, "e3x_tp_backward_w_uvw: x1, x2 and grad_out must be 16-byte aligned");
    if ((rc = prepare_mfma_dw(P))) return rc;
    if ((rc = load_dw_function(P, dev))) return rc;
    // batch slices: enough workgroups for a few waves of the chip, at least 256 rows each
    const long long wgs = P->dw_tiles * P->dw_paths;
    long long slices = (2048 + wgs - 1) / wgs;
    slices = std::min(slices, (long long)((Z + 255) / 256));
    slices = std::max(1LL, std::min(slices, 1024LL));
    long long rows_per_slice = (Z + slices - 1) / slices;
    rows_per_slice = (rows_per_slice + 95) / 96 * 96;  // whole chunks of the kernel (24 rows, or 32 on split operands)
    slices = (Z + rows_per_slice - 1) / rows_per_slice;
    int accumulate = slices > 1;
    if (accumulate && (rc = e3x::fill_zero_bytes(grad_w, (size_t)P->weight_numel * 4, st))) return rc;
    void* args[] = {(void*)&x1, (void*)&x2, (void*)&grad_out, (void*)&grad_w, (void*)&n_rows, (void*)&rows_per_slice,
                    (void*)&accumulate};
    hipError_t err = hipModuleLaunchKernel(P->dw->fn_dw[dev], (unsigned)P->dw_tiles, (unsigned)P->dw_paths,
                                           (unsigned)slices, 256, 1, 1, 0, st, args, nullptr);
    if (err != hipSuccess)
      return fail(E3X_ERR_HIP, std::string("e3x_tp_backward_w_uvw: launch failed: ") + hipGetErrorString(err));
    return E3X_OK;
  }
  if (P->shared_weights && (rc = e3x::fill_zero_bytes(grad_w, (size_t)P->weight_numel * 4, st))) return rc;
  hipFunction_t fn_dw = nullptr;
  if (node_dw_on_valu(P)) {
    if ((rc = prepare_valu_dw(P))) return rc;
    if ((rc = load_valu_dw_function(P, dev))) return rc;
    fn_dw = P->dw->fn_dw[dev];
  } else {
    if ((rc = load_functions(P, dev))) return rc;
    fn_dw = P->subs[0]->fn_dw[dev];
  }
  // one thread per (path, v, w) column of the weight blocks
  long long cols = 0;
  for (const auto& q : P->paths) cols += (long long)P->in2[q.in2].mul * P->out[q.out].mul;
  // with fewer than 256 columns a workgroup is (power of two >= columns) x (interleaved rows of its slice)
  long long cpb = 1;
  while (cpb < cols && cpb < 256) cpb *= 2;
  const long long row_lanes = 256 / cpb;
  const long long wblocks = (cols + cpb - 1) / cpb;
  // enough batch slices to fill the chip a few times over, at least 16 rows per row lane
  long long slices = (2048 + wblocks - 1) / wblocks;
  if (slices > (Z + 16 * row_lanes - 1) / (16 * row_lanes)) slices = (Z + 16 * row_lanes - 1) / (16 * row_lanes);
  if (slices < 1) slices = 1;
  if (slices > 65535) slices = 65535;
  long long rows_per_slice = (Z + slices - 1) / slices;
  slices = (Z + rows_per_slice - 1) / rows_per_slice;
  void* args[] = {(void*)&x1, (void*)&x2, (void*)&grad_out, (void*)&grad_w, (void*)&n_rows, (void*)&rows_per_slice};
  hipError_t err = hipModuleLaunchKernel(fn_dw, (unsigned)wblocks, (unsigned)slices, 1, 256, 1, 1, 0, st, args, nullptr);
  if (err != hipSuccess)
    return fail(E3X_ERR_HIP, std::string("e3x_tp_backward_w_uvw: launch failed: ") + hipGetErrorString(err));
  return E3X_OK;
}
