// The C ABI of libfta.so used from plain C++ with the HIP runtime only (no PyTorch, no Python):
// allocates device buffers, runs fta_fwd and fta_bwd on a small problem and checks O, lse, dQ, dK,
// dV and dBias against a double-precision loop implementation of the same formulas
// (S = sm_scale * q.k + bias, P = softmax_k S, O = P V; dS = P * (dP - rowsum(O * dO)), dBias = sum
// over L1 rows of dS).  Prints the largest errors and returns 0 if they are within the tolerances
// the test suite uses (O max-abs 1e-2, gradients relative-L2 1e-2).
//
//   fta_c_demo [L1 L2 D]        (defaults 3 128 32; B = 1, H = 2)
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <vector>

#include "fta.h"

namespace {

typedef _Float16 half_t;

#define HIP_OK(call)                                                                  \
  do {                                                                                \
    hipError_t e_ = (call);                                                           \
    if (e_ != hipSuccess) {                                                           \
      fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));               \
      return 2;                                                                       \
    }                                                                                 \
  } while (0)

struct Lcg {
  uint64_t s;
  double normal() {  // sum of 12 uniforms - 6: close enough to N(0,1) for test data
    double a = 0;
    for (int i = 0; i < 12; ++i) {
      s = s * 6364136223846793005ull + 1442695040888963407ull;
      a += (double)((s >> 11) & ((1ull << 53) - 1)) / (double)(1ull << 53);
    }
    return a - 6.0;
  }
};

std::vector<half_t> random_halfs(size_t n, Lcg& g, double std) {
  std::vector<half_t> v(n);
  for (size_t i = 0; i < n; ++i) v[i] = (half_t)(g.normal() * std);
  return v;
}

template <class T>
T* to_device(const std::vector<T>& h) {
  T* d = nullptr;
  if (hipMalloc(&d, h.size() * sizeof(T)) != hipSuccess) return nullptr;
  if (hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return d;
}

double rel_l2(const std::vector<half_t>& got, const std::vector<double>& ref) {
  double num = 0, den = 0;
  for (size_t i = 0; i < ref.size(); ++i) {
    const double d = (double)got[i] - ref[i];
    num += d * d;
    den += ref[i] * ref[i];
  }
  return sqrt(num / (den > 0 ? den : 1));
}

}  // namespace

int main(int argc, char** argv) {
  const int B = 1, H = 2;
  const int L1 = argc > 1 ? atoi(argv[1]) : 3, L2 = argc > 2 ? atoi(argv[2]) : 128, D = argc > 3 ? atoi(argv[3]) : 32;
  const float sm = 1.0f / sqrtf((float)D);
  const size_t n5 = (size_t)B * H * L1 * L2 * D, n4 = (size_t)B * H * L2 * L2, nl = (size_t)B * H * L1 * L2;
  printf("libfta version %d, B=%d H=%d L1=%d L2=%d D=%d\n", fta_version(), B, H, L1, L2, D);

  Lcg g{20};
  const std::vector<half_t> q = random_halfs(n5, g, 1.0), k = random_halfs(n5, g, 1.0), v = random_halfs(n5, g, 1.0),
                            bias = random_halfs(n4, g, 1.0), dout = random_halfs(n5, g, 1.0);

  // ---- reference in double precision
  std::vector<double> ro(n5), rlse(nl), rdq(n5, 0.0), rdk(n5, 0.0), rdv(n5, 0.0), rdb(n4, 0.0);
  std::vector<double> p(L2), dp(L2);
  for (int bh = 0; bh < B * H; ++bh)
    for (int i = 0; i < L1; ++i) {
      const size_t row = ((size_t)bh * L1 + i) * L2;
      for (int j = 0; j < L2; ++j) {
        double mx = -1e300;
        for (int kk = 0; kk < L2; ++kk) {
          double s = 0;
          for (int d = 0; d < D; ++d) s += (double)q[(row + j) * D + d] * (double)k[(row + kk) * D + d];
          p[kk] = s * sm + (double)bias[((size_t)bh * L2 + j) * L2 + kk];
          if (p[kk] > mx) mx = p[kk];
        }
        double l = 0;
        for (int kk = 0; kk < L2; ++kk) { p[kk] = exp(p[kk] - mx); l += p[kk]; }
        rlse[row + j] = (mx + log(l)) / log(2.0);
        double delta = 0;
        for (int d = 0; d < D; ++d) {
          double o = 0;
          for (int kk = 0; kk < L2; ++kk) o += p[kk] / l * (double)v[(row + kk) * D + d];
          ro[(row + j) * D + d] = o;
          delta += o * (double)dout[(row + j) * D + d];
        }
        for (int kk = 0; kk < L2; ++kk) {
          p[kk] /= l;
          double x = 0;
          for (int d = 0; d < D; ++d) x += (double)dout[(row + j) * D + d] * (double)v[(row + kk) * D + d];
          dp[kk] = x;
        }
        for (int kk = 0; kk < L2; ++kk) {
          const double ds = p[kk] * (dp[kk] - delta);
          rdb[((size_t)bh * L2 + j) * L2 + kk] += ds;
          for (int d = 0; d < D; ++d) {
            rdv[(row + kk) * D + d] += p[kk] * (double)dout[(row + j) * D + d];
            rdq[(row + j) * D + d] += sm * ds * (double)k[(row + kk) * D + d];
            rdk[(row + kk) * D + d] += sm * ds * (double)q[(row + j) * D + d];
          }
        }
      }
    }

  // ---- device side, through the C ABI only
  half_t *dq_in = to_device(q), *dk_in = to_device(k), *dv_in = to_device(v), *db_in = to_device(bias), *ddo = to_device(dout);
  half_t *d_o, *d_dq, *d_dk, *d_dv, *d_db;
  float* d_lse;
  void* d_ws;
  if (!dq_in || !dk_in || !dv_in || !db_in || !ddo) { fprintf(stderr, "device allocation failed\n"); return 2; }
  HIP_OK(hipMalloc(&d_o, n5 * 2)); HIP_OK(hipMalloc(&d_dq, n5 * 2)); HIP_OK(hipMalloc(&d_dk, n5 * 2)); HIP_OK(hipMalloc(&d_dv, n5 * 2));
  HIP_OK(hipMalloc(&d_db, n4 * 2)); HIP_OK(hipMalloc(&d_lse, nl * 4));
  const size_t nws = fta_bwd_workspace_bytes(B, H, L1, L2, D);
  if (nws == 0) { fprintf(stderr, "sizes not supported: %s\n", fta_strerror(FTA_ERR_SEQ_LEN)); return 2; }
  HIP_OK(hipMalloc(&d_ws, nws));
  const int64_t s5[4] = {(int64_t)H * L1 * L2 * D, (int64_t)L1 * L2 * D, (int64_t)L2 * D, D};
  const int64_t s4[3] = {(int64_t)H * L2 * L2, (int64_t)L2 * L2, L2};
  auto t5 = [&](void* ptr) { fta_tensor5 t; t.ptr = ptr; for (int i = 0; i < 4; ++i) t.stride[i] = s5[i]; return t; };
  auto t4 = [&](void* ptr) { fta_tensor4 t; t.ptr = ptr; for (int i = 0; i < 3; ++i) t.stride[i] = s4[i]; return t; };
  const fta_tensor5 tq = t5(dq_in), tk = t5(dk_in), tv = t5(dv_in), to = t5(d_o), tdo = t5(ddo), tdq = t5(d_dq), tdk = t5(d_dk),
                    tdv = t5(d_dv);
  const fta_tensor4 tb = t4(db_in), tdb = t4(d_db);
  char plan[1024];
  if (fta_describe_plan(B, H, L1, L2, D, plan, sizeof plan) == FTA_OK) printf("%s", plan);
  int rc = fta_fwd(&tq, &tk, &tv, &tb, &to, d_lse, B, H, L1, L2, D, sm, nullptr);
  if (rc != 0) { fprintf(stderr, "fta_fwd: %s\n", fta_strerror(rc)); return 2; }
  rc = fta_bwd(&tq, &tk, &tv, &tb, &to, d_lse, &tdo, &tdq, &tdk, &tdv, &tdb, d_ws, nws, B, H, L1, L2, D, sm, nullptr);
  if (rc != 0) { fprintf(stderr, "fta_bwd: %s\n", fta_strerror(rc)); return 2; }
  HIP_OK(hipDeviceSynchronize());

  std::vector<half_t> ho(n5), hdq(n5), hdk(n5), hdv(n5), hdb(n4);
  std::vector<float> hlse(nl);
  HIP_OK(hipMemcpy(ho.data(), d_o, n5 * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(hdq.data(), d_dq, n5 * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(hdk.data(), d_dk, n5 * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(hdv.data(), d_dv, n5 * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(hdb.data(), d_db, n4 * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(hlse.data(), d_lse, nl * 4, hipMemcpyDeviceToHost));

  double eo = 0, el = 0;
  for (size_t i = 0; i < n5; ++i) eo = fmax(eo, fabs((double)ho[i] - ro[i]));
  for (size_t i = 0; i < nl; ++i) el = fmax(el, fabs((double)hlse[i] - rlse[i]));
  const double rq = rel_l2(hdq, rdq), rk = rel_l2(hdk, rdk), rv = rel_l2(hdv, rdv), rb = rel_l2(hdb, rdb);
  printf("O max-abs %.3e  lse max-abs %.3e  dQ rel-L2 %.3e  dK %.3e  dV %.3e  dBias %.3e\n", eo, el, rq, rk, rv, rb);
  const bool ok = eo <= 1e-2 && el <= 1e-2 && rq <= 1e-2 && rk <= 1e-2 && rv <= 1e-2 && rb <= 1e-2;
  printf(ok ? "PASS\n" : "FAIL\n");
  return ok ? 0 : 1;
}
