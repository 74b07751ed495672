// A caller of libhbsattn_amd.so without torch or Python: block geometry on the host, device buffers
// from hipMalloc, one hbsa_fwd call on a stream, and a check against plain loops.
// Build:  hipcc -O2 -I include hbsattn_amd/csrc/cabi_example.cpp -L hbsattn_amd -lhbsattn_amd \
//               -Wl,-rpath,'$ORIGIN' -o hbsattn_amd/cabi_example      (python -m hbsattn_amd.build does it)
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "hbsattn_amd.h"

#define HIP_OK(x)                                                              \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));             \
      return 2;                                                                \
    }                                                                          \
  } while (0)

static uint16_t to_bf16(float f) {   // round to nearest even
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

int main() {
  // two packed sequences, GQA 4/2, head dim 64, 32x48 blocks, causal, a fixed pseudo-random mask
  const int32_t batch = 2, hq = 4, hk = 2, d = 64, qbs = 32, kbs = 48;
  const std::vector<int32_t> cu_q = {0, 100, 164}, cu_k = {0, 130, 194};
  int32_t nqb = 0, nkb = 0;
  std::vector<int32_t> cu_nqb(batch + 1), cu_nkb(batch + 1);
  if (hbsa_calculate_blocks(cu_q.data(), batch, qbs, &nqb, cu_nqb.data(), nullptr, nullptr, 0) ||
      hbsa_calculate_blocks(cu_k.data(), batch, kbs, &nkb, cu_nkb.data(), nullptr, nullptr, 0)) {
    std::fprintf(stderr, "hbsa_calculate_blocks: %s\n", hbsa_last_error());
    return 2;
  }
  std::vector<int32_t> cu_qb(nqb + 1), qb2b(nqb), cu_kb(nkb + 1), kb2b(nkb);
  hbsa_calculate_blocks(cu_q.data(), batch, qbs, &nqb, cu_nqb.data(), cu_qb.data(), qb2b.data(), nqb);
  hbsa_calculate_blocks(cu_k.data(), batch, kbs, &nkb, cu_nkb.data(), cu_kb.data(), kb2b.data(), nkb);

  const int total_q = cu_q.back(), total_k = cu_k.back();
  uint32_t rng = 12345u;
  auto next = [&]() { rng = rng * 1664525u + 1013904223u; return (float)((rng >> 8) & 0xffff) / 32768.f - 1.f; };
  std::vector<uint16_t> q((size_t)total_q * hq * d), k((size_t)total_k * hk * d), v(k.size());
  for (auto &x : q) x = to_bf16(next());
  for (auto &x : k) x = to_bf16(next());
  for (auto &x : v) x = to_bf16(next());
  std::vector<uint8_t> mask((size_t)hk * nqb * nkb);
  for (auto &m : mask) m = next() > -0.2f;

  uint16_t *dq, *dk, *dv, *dout;
  int32_t *dcu_q, *dcu_k, *dqb2b, *dcu_nqb, *dcu_nkb;
  uint8_t *dmask;
  void *ws;
  const size_t ws_bytes = hbsa_fwd_workspace_bytes_dtype(HBSA_DTYPE_BF16, total_q, total_k, hq, hk, d, nqb, nkb);
  HIP_OK(hipMalloc(&dq, q.size() * 2));
  HIP_OK(hipMalloc(&dk, k.size() * 2));
  HIP_OK(hipMalloc(&dv, v.size() * 2));
  HIP_OK(hipMalloc(&dout, q.size() * 2));
  HIP_OK(hipMalloc(&dcu_q, cu_q.size() * 4));
  HIP_OK(hipMalloc(&dcu_k, cu_k.size() * 4));
  HIP_OK(hipMalloc(&dqb2b, qb2b.size() * 4));
  HIP_OK(hipMalloc(&dcu_nqb, cu_nqb.size() * 4));
  HIP_OK(hipMalloc(&dcu_nkb, cu_nkb.size() * 4));
  HIP_OK(hipMalloc(&dmask, mask.size()));
  HIP_OK(hipMalloc(&ws, ws_bytes));
  HIP_OK(hipMemcpy(dq, q.data(), q.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dk, k.data(), k.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dv, v.data(), v.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dcu_q, cu_q.data(), cu_q.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dcu_k, cu_k.data(), cu_k.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dqb2b, qb2b.data(), qb2b.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dcu_nqb, cu_nqb.data(), cu_nqb.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dcu_nkb, cu_nkb.data(), cu_nkb.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dmask, mask.data(), mask.size(), hipMemcpyHostToDevice));

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  const float scale = 1.f / std::sqrt((float)d);
  const int64_t strides[11] = {(int64_t)hq * d, d, (int64_t)hk * d, d, (int64_t)hk * d, d, (int64_t)hq * d, d,
                               (int64_t)nqb * nkb, nkb, 1};
  const int rc = hbsa_fwd(dq, dk, dv, dout, dcu_q, dcu_k, dmask, dqb2b, dcu_nqb, dcu_nkb, ws, ws_bytes, HBSA_DTYPE_BF16,
                          batch, total_q, total_k, hq, hk, d, nqb, nkb, qbs, kbs, /*causal=*/1, scale, strides, stream);
  if (rc != 0) {
    std::fprintf(stderr, "hbsa_fwd failed (%d): %s\n", rc, hbsa_last_error());
    return 2;
  }
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<uint16_t> out(q.size());
  HIP_OK(hipMemcpy(out.data(), dout, out.size() * 2, hipMemcpyDeviceToHost));

  // plain loops over the same definition: key j of the sequence is visible to query i iff the mask bit
  // of their blocks is set and i + (k_len - q_len) >= j
  double max_err = 0.0;
  for (int b = 0; b < batch; ++b) {
    const int q_len = cu_q[b + 1] - cu_q[b], k_len = cu_k[b + 1] - cu_k[b];
    for (int h = 0; h < hq; ++h)
      for (int i = 0; i < q_len; ++i) {
        const int gq = cu_nqb[b] + i / qbs;
        std::vector<double> s(k_len, -INFINITY);
        double mx = -INFINITY;
        for (int j = 0; j < k_len; ++j) {
          const int gk = cu_nkb[b] + j / kbs;
          if (!mask[((size_t)(h / (hq / hk)) * nqb + gq) * nkb + gk] || i + (k_len - q_len) < j) continue;
          double acc = 0;
          for (int e = 0; e < d; ++e)
            acc += (double)from_bf16(q[((size_t)(cu_q[b] + i) * hq + h) * d + e]) *
                   from_bf16(k[((size_t)(cu_k[b] + j) * hk + h / (hq / hk)) * d + e]);
          s[j] = acc * scale;
          mx = std::max(mx, s[j]);
        }
        for (int e = 0; e < d; ++e) {
          double num = 0, den = 0;
          for (int j = 0; j < k_len; ++j) {
            if (s[j] == -INFINITY) continue;
            const double p = std::exp(s[j] - mx);
            den += p;
            num += p * from_bf16(v[((size_t)(cu_k[b] + j) * hk + h / (hq / hk)) * d + e]);
          }
          const double ref = den > 0 ? num / den : 0.0;
          max_err = std::max(max_err, std::fabs(ref - from_bf16(out[((size_t)(cu_q[b] + i) * hq + h) * d + e])));
        }
      }
  }
  std::printf("hbsa_fwd through the C ABI: %d q blocks, %d k blocks, max |error| against plain loops %.3e\n", nqb, nkb,
              max_err);
  return max_err <= 2e-2 ? 0 : 1;
}
