// Host-side real-basis Wigner 3j tensors.
//
// Same construction as the reference (e3nn/o3/_wigner.py:150-164): Condon-Shortley
// SU(2) Clebsch-Gordan coefficients (Racah's single-sum formula), a unitary change of
// basis real -> complex per index (:30-41), real part, Frobenius normalisation.
// Factorials are carried in long double (exact through 25!, 64-bit mantissa above).
#include <cmath>
#include <complex>
#include <mutex>
#include <map>
#include <tuple>
#include <vector>

#include "e3x_internal.h"

namespace e3x {

static long double fact(int n) {
  static long double table[80];
  static bool init = false;
  if (!init) {
    table[0] = 1.0L;
    for (int i = 1; i < 80; ++i) table[i] = table[i - 1] * (long double)i;
    init = true;
  }
  return table[n];
}

// <j1 m1 j2 m2 | j3 m3>
static long double su2_cg(int j1, int m1, int j2, int m2, int j3, int m3) {
  if (m3 != m1 + m2 || j3 < std::abs(j1 - j2) || j3 > j1 + j2) return 0.0L;
  long double pref = (long double)(2 * j3 + 1) * fact(j3 + j1 - j2) * fact(j3 - j1 + j2) * fact(j1 + j2 - j3) /
                     fact(j1 + j2 + j3 + 1);
  pref *= fact(j3 + m3) * fact(j3 - m3) * fact(j1 - m1) * fact(j1 + m1) * fact(j2 - m2) * fact(j2 + m2);
  long double s = 0.0L;
  for (int k = 0; k <= j1 + j2 - j3; ++k) {
    int a[6] = {k, j1 + j2 - j3 - k, j1 - m1 - k, j2 + m2 - k, j3 - j2 + m1 + k, j3 - j1 - m2 + k};
    bool ok = true;
    long double d = 1.0L;
    for (int t = 0; t < 6; ++t) {
      if (a[t] < 0) { ok = false; break; }
      d *= fact(a[t]);
    }
    if (ok) s += ((k & 1) ? -1.0L : 1.0L) / d;
  }
  return sqrtl(pref) * s;
}

typedef std::complex<long double> cld;

// q[row = complex index l+m][col = real index]
static std::vector<cld> real_to_complex(int l) {
  const int d = 2 * l + 1;
  std::vector<cld> q(d * d, cld(0, 0));
  const long double r = 1.0L / sqrtl(2.0L);
  for (int m = 1; m <= l; ++m) {
    const long double sg = (m & 1) ? -1.0L : 1.0L;
    q[(l - m) * d + (l + m)] = cld(r, 0);
    q[(l - m) * d + (l - m)] = cld(0, -r);
    q[(l + m) * d + (l + m)] = cld(sg * r, 0);
    q[(l + m) * d + (l - m)] = cld(0, sg * r);
  }
  q[l * d + l] = cld(1, 0);
  // times (-i)^l so that the resulting coupling tensor is real
  cld ph(1, 0);
  for (int t = 0; t < l; ++t) ph *= cld(0, -1);
  for (auto& v : q) v *= ph;
  return q;
}

const std::vector<double>& wigner_3j(int l1, int l2, int l3) {
  static std::mutex mu;
  static std::map<std::tuple<int, int, int>, std::vector<double>> cache;
  std::lock_guard<std::mutex> lock(mu);
  auto key = std::make_tuple(l1, l2, l3);
  auto it = cache.find(key);
  if (it != cache.end()) return it->second;

  const int d1 = 2 * l1 + 1, d2 = 2 * l2 + 1, d3 = 2 * l3 + 1;
  std::vector<long double> c(d1 * d2 * d3, 0.0L);
  for (int m1 = -l1; m1 <= l1; ++m1)
    for (int m2 = -l2; m2 <= l2; ++m2) {
      int m3 = m1 + m2;
      if (std::abs(m3) <= l3) c[((l1 + m1) * d2 + (l2 + m2)) * d3 + (l3 + m3)] = su2_cg(l1, m1, l2, m2, l3, m3);
    }
  auto q1 = real_to_complex(l1), q2 = real_to_complex(l2), q3 = real_to_complex(l3);
  // R[j,l,m] = sum_{i,k,n} q1[i,j] q2[k,l] conj(q3[n,m]) c[i,k,n]
  std::vector<long double> r(d1 * d2 * d3, 0.0L);
  long double nrm = 0.0L;
  for (int j = 0; j < d1; ++j)
    for (int l = 0; l < d2; ++l)
      for (int m = 0; m < d3; ++m) {
        cld acc(0, 0);
        for (int i = 0; i < d1; ++i) {
          if (q1[i * d1 + j] == cld(0, 0)) continue;
          for (int k = 0; k < d2; ++k) {
            if (q2[k * d2 + l] == cld(0, 0)) continue;
            int n = i + k - l1 - l2 + l3;  // m3 = m1 + m2
            if (n < 0 || n >= d3) continue;
            acc += q1[i * d1 + j] * q2[k * d2 + l] * std::conj(q3[n * d3 + m]) * c[(i * d2 + k) * d3 + n];
          }
        }
        r[(j * d2 + l) * d3 + m] = acc.real();
        nrm += acc.real() * acc.real();
      }
  nrm = sqrtl(nrm);
  std::vector<double> out(d1 * d2 * d3);
  for (size_t t = 0; t < out.size(); ++t) {
    long double v = r[t] / nrm;
    out[t] = (fabsl(v) < 1e-15L) ? 0.0 : (double)v;
  }
  return cache.emplace(key, std::move(out)).first->second;
}

}  // namespace e3x

extern "C" int e3x_wigner_3j(int l1, int l2, int l3, double* out) {
  if (l1 < 0 || l2 < 0 || l3 < 0 || l1 + l2 + l3 + 1 >= 80 || l3 < std::abs(l1 - l2) || l3 > l1 + l2 || !out)
    return e3x::fail(E3X_ERR_INVALID, "e3x_wigner_3j: need |l1-l2| <= l3 <= l1+l2 and l1+l2+l3 < 79");
  const auto& c = e3x::wigner_3j(l1, l2, l3);
  for (size_t i = 0; i < c.size(); ++i) out[i] = c[i];
  return E3X_OK;
}
