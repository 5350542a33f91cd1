// Torch-free caller of the C ABI in include/mi355x_rownorm.h: what a host that only has
// device pointers (a C++ runtime, a cgo/JNI/ctypes binding) does.  The role the reference's
// test/sycl/main.cpp plays there: a build-and-run check below the framework.
//
//   cabi_check <path/to/libmi355x_rownorm.so> symbols   no GPU: every declared symbol resolves,
//                                                        arguments are validated before launch
//   cabi_check <path/to/libmi355x_rownorm.so> gpu       one small call of each operator family
//                                                        on device memory from hipMalloc, checked
//                                                        against double-precision closed forms
//
// The library is opened with dlopen so that this file links against nothing but libdl and the
// HIP runtime.
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/mi355x_rownorm.h"

#define DECL(name) decltype(&name) p_##name = nullptr
DECL(mi355x_rownorm_error_string);
DECL(mi355x_rownorm_abi_version);
DECL(mi355x_layer_norm_fwd);
DECL(mi355x_layer_norm_bwd_workspace_bytes);
DECL(mi355x_layer_norm_bwd);
DECL(mi355x_rms_norm_fwd);
DECL(mi355x_rms_norm_bwd_workspace_bytes);
DECL(mi355x_rms_norm_bwd);
DECL(mi355x_rms_norm_bwd_static_limit_bytes);
DECL(mi355x_rms_norm_bwd_static);
DECL(mi355x_add_layer_norm_fwd);
DECL(mi355x_add_rms_norm_fwd);
DECL(mi355x_add_layer_norm_bwd);
DECL(mi355x_add_rms_norm_bwd);
DECL(mi355x_softmax_fwd);
DECL(mi355x_softmax_bwd);
DECL(mi355x_safe_softmax_fwd);
DECL(mi355x_masked_softmax_fwd);
DECL(mi355x_masked_softmax_bwd);
DECL(mi355x_softmax_strided_fwd);
DECL(mi355x_softmax_strided_bwd);
DECL(mi355x_softmax_strided_plan);
DECL(mi355x_group_norm_fwd);
DECL(mi355x_group_norm_bwd_workspace_bytes);
DECL(mi355x_group_norm_bwd);
DECL(mi355x_group_norm_plan);
DECL(mi355x_rownorm_plan);
DECL(mi355x_rownorm_plan_at);
DECL(mi355x_rownorm_set_override);

static int failures = 0;
#define CHECK(cond)                                                       \
  do {                                                                    \
    if (!(cond)) {                                                        \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);       \
      ++failures;                                                         \
    }                                                                     \
  } while (0)
#define HIP_OK(call) CHECK((call) == hipSuccess)

template <class F>
static bool load(void* lib, const char* name, F& fn) {
  fn = reinterpret_cast<F>(dlsym(lib, name));
  if (!fn) std::printf("missing symbol %s\n", name);
  return fn != nullptr;
}

static bool load_all(void* lib) {
  bool ok = true;
#define LOAD(name) ok = load(lib, #name, p_##name) && ok
  LOAD(mi355x_rownorm_error_string);
  LOAD(mi355x_rownorm_abi_version);
  LOAD(mi355x_layer_norm_fwd);
  LOAD(mi355x_layer_norm_bwd_workspace_bytes);
  LOAD(mi355x_layer_norm_bwd);
  LOAD(mi355x_rms_norm_fwd);
  LOAD(mi355x_rms_norm_bwd_workspace_bytes);
  LOAD(mi355x_rms_norm_bwd);
  LOAD(mi355x_rms_norm_bwd_static_limit_bytes);
  LOAD(mi355x_rms_norm_bwd_static);
  LOAD(mi355x_add_layer_norm_fwd);
  LOAD(mi355x_add_rms_norm_fwd);
  LOAD(mi355x_add_layer_norm_bwd);
  LOAD(mi355x_add_rms_norm_bwd);
  LOAD(mi355x_softmax_fwd);
  LOAD(mi355x_softmax_bwd);
  LOAD(mi355x_safe_softmax_fwd);
  LOAD(mi355x_masked_softmax_fwd);
  LOAD(mi355x_masked_softmax_bwd);
  LOAD(mi355x_softmax_strided_fwd);
  LOAD(mi355x_softmax_strided_bwd);
  LOAD(mi355x_softmax_strided_plan);
  LOAD(mi355x_group_norm_fwd);
  LOAD(mi355x_group_norm_bwd_workspace_bytes);
  LOAD(mi355x_group_norm_bwd);
  LOAD(mi355x_group_norm_plan);
  LOAD(mi355x_rownorm_plan);
  LOAD(mi355x_rownorm_plan_at);
  LOAD(mi355x_rownorm_set_override);
  return ok;
}

static void check_validation() {
  CHECK(p_mi355x_rownorm_abi_version() == 1);
  CHECK(std::strcmp(p_mi355x_rownorm_error_string(0), "success") == 0);
  void* one = reinterpret_cast<void*>(256);  // never dereferenced: every call below is rejected
  CHECK(p_mi355x_rms_norm_fwd(one, nullptr, one, nullptr, 4, 8, 1e-6f, (rownorm_dtype)7, ROWNORM_F32,
                              nullptr) == ROWNORM_ERR_DTYPE);
  CHECK(p_mi355x_rms_norm_fwd(one, nullptr, one, nullptr, -4, 8, 1e-6f, ROWNORM_F32, ROWNORM_F32,
                              nullptr) == ROWNORM_ERR_SHAPE);
  CHECK(p_mi355x_rms_norm_fwd(nullptr, nullptr, one, nullptr, 4, 8, 1e-6f, ROWNORM_F32, ROWNORM_F32,
                              nullptr) == ROWNORM_ERR_NULL);
  CHECK(p_mi355x_rms_norm_fwd(nullptr, nullptr, nullptr, nullptr, 0, 8, 1e-6f, ROWNORM_F32,
                              ROWNORM_F32, nullptr) == ROWNORM_OK);
  CHECK(p_mi355x_rms_norm_bwd(one, one, (const float*)one, nullptr, one, one, nullptr, 0, 4, 8,
                              ROWNORM_F32, ROWNORM_F32, nullptr) == ROWNORM_ERR_WORKSPACE);
  CHECK(p_mi355x_masked_softmax_fwd(one, one, one, 8, 16, 7, 1, 1, 1, ROWNORM_F32, nullptr) ==
        ROWNORM_ERR_SHAPE);
  CHECK(p_mi355x_group_norm_fwd(one, nullptr, nullptr, one, nullptr, nullptr, 2, 6, 4, 4, 1e-5f,
                                ROWNORM_F32, ROWNORM_F32, nullptr) == ROWNORM_ERR_SHAPE);
  rownorm_plan plan;
  CHECK(p_mi355x_rownorm_plan(ROWNORM_OP_RMS_NORM_BWD, 16384, 4096, ROWNORM_BF16, ROWNORM_BF16,
                              &plan) == 0);
  CHECK(plan.resident == 1 && plan.lanes_per_row * plan.packs_per_lane * 8 >= 4096);
  // (the query covers calls with and without dX, which may take different grids)
  CHECK(p_mi355x_rms_norm_bwd_workspace_bytes(16384, 4096, ROWNORM_BF16, ROWNORM_BF16, 1) >=
        (size_t)plan.partial_rows * 4096 * sizeof(float));
  CHECK(p_mi355x_rownorm_plan(ROWNORM_OP_RMS_NORM_BWD, 16384, 4096, ROWNORM_F32, ROWNORM_F32,
                              &plan) == 0);
  CHECK(p_mi355x_rms_norm_bwd_workspace_bytes(16384, 4096, ROWNORM_F32, ROWNORM_F32, 1) ==
        (size_t)plan.partial_rows * 4096 * sizeof(float));
}

struct DeviceBuffer {
  void* p = nullptr;
  explicit DeviceBuffer(size_t bytes) { HIP_OK(hipMalloc(&p, bytes ? bytes : 1)); }
  ~DeviceBuffer() { (void)hipFree(p); }
  void upload(const std::vector<float>& h) {
    HIP_OK(hipMemcpy(p, h.data(), h.size() * sizeof(float), hipMemcpyHostToDevice));
  }
  std::vector<float> download(size_t n) const {
    std::vector<float> h(n);
    HIP_OK(hipMemcpy(h.data(), p, n * sizeof(float), hipMemcpyDeviceToHost));
    return h;
  }
};

static std::vector<float> pseudo_random(size_t n, uint32_t seed, float scale) {
  std::vector<float> v(n);
  uint32_t s = seed;
  for (size_t i = 0; i < n; ++i) {
    s = s * 1664525u + 1013904223u;
    v[i] = scale * ((float)(s >> 8) / 8388608.0f - 1.0f);  // uniform in [-scale, scale)
  }
  return v;
}

static void expect_close(const std::vector<float>& got, const std::vector<double>& want,
                         const char* what) {
  double worst = 0;
  for (size_t i = 0; i < want.size(); ++i) {
    const double tol = 1e-5 + 1e-5 * std::fabs(want[i]);
    worst = std::fmax(worst, std::fabs((double)got[i] - want[i]) / tol);
  }
  std::printf("%-28s max error %.3f x (rtol = atol = 1e-5)\n", what, worst);
  CHECK(worst <= 1.0);
}

static void check_gpu() {
  int ndev = 0;
  HIP_OK(hipGetDeviceCount(&ndev));
  CHECK(ndev >= 1);
  if (ndev < 1) return;
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  const int64_t M = 37, N = 1000;
  const std::vector<float> x = pseudo_random(M * N, 1, 2.0f), dy = pseudo_random(M * N, 2, 1.0f);
  std::vector<float> w = pseudo_random(N, 3, 0.2f), b = pseudo_random(N, 4, 0.2f);
  for (auto& v : w) v += 1.0f;
  DeviceBuffer dx_(M * N * 4), ddy(M * N * 4), dw(N * 4), db(N * 4), dyo(M * N * 4), dmean(M * 4),
      drstd(M * 4), dgx(M * N * 4), dgw(N * 4);
  dx_.upload(x);
  ddy.upload(dy);
  dw.upload(w);
  db.upload(b);

  // _fused_rms_norm forward + backward
  CHECK(p_mi355x_rms_norm_fwd(dx_.p, dw.p, dyo.p, (float*)drstd.p, M, N, 1e-6f, ROWNORM_F32,
                              ROWNORM_F32, stream) == 0);
  const size_t ws_bytes = p_mi355x_rms_norm_bwd_workspace_bytes(M, N, ROWNORM_F32, ROWNORM_F32, 1);
  DeviceBuffer ws(ws_bytes);
  CHECK(p_mi355x_rms_norm_bwd(ddy.p, dx_.p, (float*)drstd.p, dw.p, dgx.p, dgw.p, ws.p, ws_bytes, M, N,
                              ROWNORM_F32, ROWNORM_F32, stream) == 0);
  HIP_OK(hipStreamSynchronize(stream));
  {
    std::vector<double> y(M * N), gx(M * N), gw(N, 0.0);
    for (int64_t r = 0; r < M; ++r) {
      double ss = 0;
      for (int64_t j = 0; j < N; ++j) ss += (double)x[r * N + j] * x[r * N + j];
      const double rs = 1.0 / std::sqrt(ss / N + 1e-6);
      double s2 = 0;
      for (int64_t j = 0; j < N; ++j) {
        y[r * N + j] = x[r * N + j] * rs * w[j];
        s2 += (double)dy[r * N + j] * w[j] * x[r * N + j] * rs;
        gw[j] += (double)dy[r * N + j] * x[r * N + j] * rs;
      }
      for (int64_t j = 0; j < N; ++j)
        gx[r * N + j] = (rs / N) * (N * (double)dy[r * N + j] * w[j] - x[r * N + j] * rs * s2);
    }
    expect_close(dyo.download(M * N), y, "rms_norm forward");
    expect_close(dgx.download(M * N), gx, "rms_norm backward dx");
    expect_close(dgw.download(N), gw, "rms_norm backward dweight");
  }

  // native_layer_norm forward
  CHECK(p_mi355x_layer_norm_fwd(dx_.p, dw.p, db.p, dyo.p, (float*)dmean.p, (float*)drstd.p, M, N, 1e-5f,
                                ROWNORM_F32, ROWNORM_F32, stream) == 0);
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<double> mu(M), rs(M);
  {
    std::vector<double> y(M * N);
    for (int64_t r = 0; r < M; ++r) {
      double s = 0, v = 0;
      for (int64_t j = 0; j < N; ++j) s += x[r * N + j];
      mu[r] = s / N;
      for (int64_t j = 0; j < N; ++j) v += (x[r * N + j] - mu[r]) * (x[r * N + j] - mu[r]);
      rs[r] = 1.0 / std::sqrt(v / N + 1e-5);
      for (int64_t j = 0; j < N; ++j) y[r * N + j] = (x[r * N + j] - mu[r]) * rs[r] * w[j] + b[j];
    }
    expect_close(dyo.download(M * N), y, "layer_norm forward");
    expect_close(dmean.download(M), mu, "layer_norm mean");
    expect_close(drstd.download(M), rs, "layer_norm rstd");
  }

  // _softmax forward over the innermost dimension, and over the middle one of [M, 25, 40]
  CHECK(p_mi355x_softmax_fwd(dx_.p, dyo.p, M, N, ROWNORM_F32, ROWNORM_F32, 0, stream) == 0);
  HIP_OK(hipStreamSynchronize(stream));
  {
    std::vector<double> y(M * N);
    for (int64_t r = 0; r < M; ++r) {
      double m = -INFINITY, s = 0;
      for (int64_t j = 0; j < N; ++j) m = std::fmax(m, (double)x[r * N + j]);
      for (int64_t j = 0; j < N; ++j) s += std::exp(x[r * N + j] - m);
      for (int64_t j = 0; j < N; ++j) y[r * N + j] = std::exp(x[r * N + j] - m) / s;
    }
    expect_close(dyo.download(M * N), y, "softmax forward");
  }
  CHECK(p_mi355x_softmax_strided_fwd(dx_.p, dyo.p, M, 25, 40, ROWNORM_F32, ROWNORM_F32, ROWNORM_SOFTMAX,
                                     stream) == 0);
  HIP_OK(hipStreamSynchronize(stream));
  {
    std::vector<double> y(M * N);
    for (int64_t o = 0; o < M; ++o)
      for (int64_t i = 0; i < 40; ++i) {
        double m = -INFINITY, s = 0;
        for (int64_t d = 0; d < 25; ++d) m = std::fmax(m, (double)x[(o * 25 + d) * 40 + i]);
        for (int64_t d = 0; d < 25; ++d) s += std::exp(x[(o * 25 + d) * 40 + i] - m);
        for (int64_t d = 0; d < 25; ++d)
          y[(o * 25 + d) * 40 + i] = std::exp(x[(o * 25 + d) * 40 + i] - m) / s;
      }
    expect_close(dyo.download(M * N), y, "softmax forward, dim 1 of 3");
  }

  // native_group_norm forward: [M, 20, 50] in 4 groups of 5 channels
  {
    const int64_t C = 20, HxW = 50, G = 4, D = C / G, L = D * HxW;
    DeviceBuffer gmean(M * G * 4), grstd(M * G * 4);
    CHECK(p_mi355x_group_norm_fwd(dx_.p, dw.p, db.p, dyo.p, gmean.p, grstd.p, M, C, HxW, G, 1e-5f,
                                  ROWNORM_F32, ROWNORM_F32, stream) == 0);
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<double> y(M * N);
    for (int64_t r = 0; r < M * G; ++r) {
      double s = 0, v = 0;
      for (int64_t p = 0; p < L; ++p) s += x[r * L + p];
      const double m = s / L;
      for (int64_t p = 0; p < L; ++p) v += (x[r * L + p] - m) * (x[r * L + p] - m);
      const double rstd = 1.0 / std::sqrt(v / L + 1e-5);
      for (int64_t p = 0; p < L; ++p) {
        const int64_t c = (r % G) * D + p / HxW;
        y[r * L + p] = (x[r * L + p] - m) * rstd * w[c] + b[c];
      }
    }
    expect_close(dyo.download(M * N), y, "group_norm forward");
  }
  HIP_OK(hipStreamDestroy(stream));
}

int main(int argc, char** argv) {
  if (argc != 3) {
    std::printf("usage: %s <libmi355x_rownorm.so> symbols|gpu\n", argv[0]);
    return 2;
  }
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!lib) {
    std::printf("cannot load %s: %s\n", argv[1], dlerror());
    return 1;
  }
  if (!load_all(lib)) return 1;
  check_validation();
  if (std::strcmp(argv[2], "gpu") == 0) check_gpu();
  std::printf(failures ? "cabi_check: %d check(s) FAILED\n" : "cabi_check: ok\n", failures);
  return failures ? 1 : 0;
}
