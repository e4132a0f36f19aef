// A caller of the C ABI written against include/jvpfa.h and the HIP runtime only: no Python, no
// torch.  It allocates device memory itself, runs the fused dual forward and the backward of
// <gO,O> + <gT,O'> on a small fp32 problem (boolean key-padding mask, then causal), and compares
// with a direct O(L^2) evaluation in double precision written out below.  Test infrastructure:
// built by jvp_flash_attention_amd/build.py next to the library and run by the GPU tests.
//
// The dense evaluation follows the definitions the reference's kernels implement
// (jvp_flash_attention/jvp_attention.py:232-336 for O and O', :1541-1553 and :1687-1697 for the
// first-order gradients) plus the tangent-path terms.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "jvpfa.h"

#define HIP_OK(x)                                                                  \
  do {                                                                             \
    hipError_t e_ = (x);                                                           \
    if (e_ != hipSuccess) {                                                        \
      std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                 \
      std::exit(2);                                                                \
    }                                                                              \
  } while (0)

namespace {

constexpr int Z = 2, H = 2, L = 80, D = 64;
constexpr size_t N = (size_t)Z * H * L * D;

struct Lcg {  // small deterministic generator, roughly N(0,1) by summing uniforms
  uint64_t s;
  double uni() {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return (double)(s >> 11) / 9007199254740992.0;
  }
  float normal() {
    double a = 0;
    for (int i = 0; i < 12; ++i) a += uni();
    return (float)(a - 6.0);
  }
};

template <typename T> T *to_device(const std::vector<T> &h) {
  T *d = nullptr;
  HIP_OK(hipMalloc(reinterpret_cast<void **>(&d), h.size() * sizeof(T)));
  HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
  return d;
}
template <typename T> T *device_buffer(size_t n) {
  T *d = nullptr;
  HIP_OK(hipMalloc(reinterpret_cast<void **>(&d), n * sizeof(T)));
  return d;
}
std::vector<float> to_host(const float *d, size_t n) {
  std::vector<float> h(n);
  HIP_OK(hipMemcpy(h.data(), d, n * sizeof(float), hipMemcpyDeviceToHost));
  return h;
}

struct Dense {  // everything in double, (Z, H, L, D) row-major
  std::vector<double> O, Ot, dq, dk, dv;
};

// keep(z, i, j): may query i of batch z attend key j
template <typename Keep>
Dense dense(const std::vector<float> &q, const std::vector<float> &k, const std::vector<float> &v,
            const std::vector<float> &qt, const std::vector<float> &kt, const std::vector<float> &vt,
            const std::vector<float> &go, const std::vector<float> &gt, double scale, Keep keep) {
  Dense r;
  r.O.assign(N, 0), r.Ot.assign(N, 0), r.dq.assign(N, 0), r.dk.assign(N, 0), r.dv.assign(N, 0);
  std::vector<double> s(L), sp(L), p(L), pp(L);
  for (int z = 0; z < Z; ++z)
    for (int h = 0; h < H; ++h) {
      const size_t base = ((size_t)z * H + h) * L * D;
      for (int i = 0; i < L; ++i) {
        const float *qi = &q[base + (size_t)i * D], *qti = &qt[base + (size_t)i * D];
        double m = -INFINITY;
        for (int j = 0; j < L; ++j) {
          const float *kj = &k[base + (size_t)j * D], *ktj = &kt[base + (size_t)j * D];
          double a = 0, b = 0;
          for (int d = 0; d < D; ++d) {
            a += (double)qi[d] * kj[d];
            b += (double)qti[d] * kj[d] + (double)qi[d] * ktj[d];
          }
          s[j] = keep(z, i, j) ? a * scale : -INFINITY;
          sp[j] = b * scale;
          m = std::fmax(m, s[j]);
        }
        double l = 0, mu = 0;
        for (int j = 0; j < L; ++j) {
          p[j] = std::isinf(s[j]) ? 0.0 : std::exp(s[j] - m);
          l += p[j];
        }
        for (int j = 0; j < L; ++j) {
          p[j] /= l;
          mu += p[j] * sp[j];
        }
        for (int j = 0; j < L; ++j) pp[j] = p[j] * (sp[j] - mu);  // tangent of p
        double *Oi = &r.O[base + (size_t)i * D], *Oti = &r.Ot[base + (size_t)i * D];
        for (int j = 0; j < L; ++j)
          for (int d = 0; d < D; ++d) {
            Oi[d] += p[j] * v[base + (size_t)j * D + d];
            Oti[d] += pp[j] * v[base + (size_t)j * D + d] + p[j] * vt[base + (size_t)j * D + d];
          }
        // backward of <gO,O> + <gT,O'> w.r.t. q, k, v through p and p' (tangent inputs held fixed)
        const float *goi = &go[base + (size_t)i * D], *gti = &gt[base + (size_t)i * D];
        std::vector<double> gp(L), gpp(L);  // dLoss/dp_j, dLoss/dp'_j
        for (int j = 0; j < L; ++j) {
          double a = 0, b = 0, c = 0;
          for (int d = 0; d < D; ++d) {
            a += (double)goi[d] * v[base + (size_t)j * D + d];
            b += (double)gti[d] * v[base + (size_t)j * D + d];
            c += (double)gti[d] * vt[base + (size_t)j * D + d];
          }
          gpp[j] = b;
          gp[j] = a + c;
          for (int d = 0; d < D; ++d) r.dv[base + (size_t)j * D + d] += p[j] * goi[d] + pp[j] * gti[d];
        }
        // p' = p (s' - mu), mu = sum p s'  =>  dLoss/dp += gpp (s' - mu) - (sum gpp p) s',  dLoss/ds' = p (gpp - sum gpp p)
        double gpp_p = 0;
        for (int j = 0; j < L; ++j) gpp_p += gpp[j] * p[j];
        std::vector<double> gs(L), gsp(L);
        double dot = 0;
        for (int j = 0; j < L; ++j) {
          gp[j] += gpp[j] * (sp[j] - mu) - gpp_p * sp[j];
          gsp[j] = p[j] * (gpp[j] - gpp_p);
          dot += gp[j] * p[j];
        }
        for (int j = 0; j < L; ++j) gs[j] = p[j] * (gp[j] - dot);  // softmax backward
        for (int j = 0; j < L; ++j)
          for (int d = 0; d < D; ++d) {
            const size_t jd = base + (size_t)j * D + d, id = base + (size_t)i * D + d;
            r.dq[id] += scale * (gs[j] * k[jd] + gsp[j] * kt[jd]);
            r.dk[jd] += scale * (gs[j] * q[id] + gsp[j] * qt[id]);
          }
      }
    }
  return r;
}

double max_abs_diff(const std::vector<float> &got, const std::vector<double> &want) {
  double e = 0;
  for (size_t i = 0; i < got.size(); ++i) e = std::fmax(e, std::fabs((double)got[i] - want[i]));
  return e;
}

}  // namespace

int main() {
  if (jvpfa_abi_version() != JVPFA_ABI_VERSION) {
    std::fprintf(stderr, "library ABI %d, header %d\n", jvpfa_abi_version(), JVPFA_ABI_VERSION);
    return 2;
  }
  Lcg rng{12345};
  std::vector<float> q(N), k(N), v(N), qt(N), kt(N), vt(N), go(N), gt(N);
  for (auto *t : {&q, &k, &v, &qt, &kt, &vt, &go, &gt})
    for (auto &x : *t) x = rng.normal();
  const int valid[Z] = {L, 47};  // key padding: batch entry 1 attends its first 47 keys
  std::vector<uint8_t> mask((size_t)Z * L);
  for (int z = 0; z < Z; ++z)
    for (int j = 0; j < L; ++j) mask[(size_t)z * L + j] = j < valid[z];

  float *dq_ = to_device(q), *dk_ = to_device(k), *dv_ = to_device(v), *dqt = to_device(qt), *dkt = to_device(kt),
        *dvt = to_device(vt), *dgo = to_device(go), *dgt = to_device(gt);
  uint8_t *dmask = to_device(mask);
  float *o = device_buffer<float>(N), *ot = device_buffer<float>(N), *M = device_buffer<float>((size_t)Z * H * L),
        *mu = device_buffer<float>((size_t)Z * H * L), *gq = device_buffer<float>(N), *gk = device_buffer<float>(N),
        *gv = device_buffer<float>(N);
  void *ws = nullptr;
  HIP_OK(hipMalloc(&ws, jvpfa_bwd_workspace_bytes(Z, H, L)));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  const double scale = 1.0 / std::sqrt((double)D);
  int failures = 0;
  for (int pass = 0; pass < 2; ++pass) {  // 0: boolean key-padding mask, 1: causal
    jvpfa_problem p{};
    p.Z = Z, p.H = H, p.L = L, p.D = D;
    p.dtype = JVPFA_FP32;
    p.causal = pass == 1;
    p.sm_scale = (float)scale;
    if (pass == 0) {
      p.mask_kind = JVPFA_MASK_BOOL;
      p.mask = dmask;
      p.mask_stride[0] = L, p.mask_stride[1] = 0, p.mask_stride[2] = 0, p.mask_stride[3] = 1;
    }
    jvpfa_fwd_args f{};
    f.struct_size = sizeof f;
    f.p = p;
    f.q = dq_, f.k = dk_, f.v = dv_, f.qt = dqt, f.kt = dkt, f.vt = dvt;
    f.o = o, f.ot = ot, f.M = M, f.mu = mu;
    int rc = jvpfa_fwd(&f, stream);
    if (rc != JVPFA_OK) {
      std::fprintf(stderr, "jvpfa_fwd: %s\n", jvpfa_error_string(rc));
      return 1;
    }
    jvpfa_bwd_args b{};
    b.struct_size = sizeof b;
    b.p = p;
    b.q = dq_, b.k = dk_, b.v = dv_, b.qt = dqt, b.kt = dkt, b.vt = dvt;
    b.o = o, b.ot = ot, b.M = M, b.mu = mu, b.go = dgo, b.gt = dgt;
    b.dq = gq, b.dk = gk, b.dv = gv;
    b.workspace = ws;
    rc = jvpfa_bwd(&b, stream);
    if (rc != JVPFA_OK) {
      std::fprintf(stderr, "jvpfa_bwd: %s\n", jvpfa_error_string(rc));
      return 1;
    }
    HIP_OK(hipStreamSynchronize(stream));
    const Dense ref = pass == 0 ? dense(q, k, v, qt, kt, vt, go, gt, scale, [&](int z, int, int j) { return j < valid[z]; })
                                : dense(q, k, v, qt, kt, vt, go, gt, scale, [](int, int i, int j) { return j <= i; });
    const struct { const char *name; const float *dev; const std::vector<double> *want; } checks[] = {
        {"O", o, &ref.O}, {"O'", ot, &ref.Ot}, {"dq", gq, &ref.dq}, {"dk", gk, &ref.dk}, {"dv", gv, &ref.dv}};
    for (const auto &c : checks) {
      const double e = max_abs_diff(to_host(c.dev, N), *c.want);
      std::printf("%s %-3s max-abs error %.3e\n", pass == 0 ? "key-padding" : "causal     ", c.name, e);
      if (!(e <= 1e-4)) ++failures;  // the fp32 bar
    }
  }
  // an argument error comes back as a status, not as a fault
  jvpfa_fwd_args bad{};
  bad.struct_size = sizeof bad;
  bad.p.Z = 1, bad.p.H = 1, bad.p.L = 32, bad.p.D = 48;
  if (jvpfa_fwd(&bad, stream) != JVPFA_E_SHAPE) ++failures;
  std::printf(failures ? "FAILED (%d)\n" : "host check ok\n", failures);
  return failures ? 1 : 0;
}
