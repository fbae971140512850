// The prefill step through the C ABI from a process with no Python and no PyTorch in it: two ragged sequences, a striped
// ring step (sp_peers = 3) with the causal boundary inside the KV chunk, GQA 8/2, fp16, checked against a double-precision
// loop on the host; then the same rows once more through lsattn_prefill_step_accumulate (the merge of a partial with
// itself: same O, LSE + ln 2).  Built by loongserve_amd/build.py; run by tests/test_gpu_c_abi.py.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "lsattn.h"

#define HIP_OK(x)                                                                         \
  do {                                                                                    \
    hipError_t e_ = (x);                                                                  \
    if (e_ != hipSuccess) {                                                               \
      fprintf(stderr, "%s:%d %s -> %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
      return 2;                                                                           \
    }                                                                                     \
  } while (0)

static uint16_t to_half(float f) {  // round to nearest even; the generator below produces small normal values only
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const int32_t exp = (int32_t)((x >> 23) & 0xff) - 127 + 15;
  const uint32_t man = x & 0x7fffffu;
  if (exp <= 0) return (uint16_t)sign;
  if (exp >= 31) return (uint16_t)(sign | 0x7c00u);
  uint32_t h = sign | ((uint32_t)exp << 10) | (man >> 13);
  const uint32_t rest = man & 0x1fffu;
  if (rest > 0x1000u || (rest == 0x1000u && (h & 1))) h++;
  return (uint16_t)h;
}
static float from_half(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, man = h & 0x3ffu;
  const uint32_t x = exp == 0 ? sign : sign | ((exp - 15 + 127) << 23) | (man << 13);
  float f;
  memcpy(&f, &x, 4);
  return f;
}
static uint64_t rng_state = 0x2545F4914F6CDD1Dull;
static float uniform() {
  rng_state ^= rng_state >> 12;
  rng_state ^= rng_state << 25;
  rng_state ^= rng_state >> 27;
  return (float)((double)((rng_state * 0x2545F4914F6CDD1Dull) >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}

int main() {
  const int Hq = 8, Hkv = 2, D = 128, B = 2, P = 3;
  const int32_t q_len[B] = {300, 77}, q_start[B] = {0, 300}, q_first[B] = {400 * P + 1, 2};
  const int32_t kv_len[B] = {700, 130}, kv_start[B] = {0, 700}, kv_first[B] = {0, 1};
  const int Tq = 377, Tk = 830;
  std::vector<uint16_t> q((size_t)Tq * Hq * D), kv((size_t)Tk * 2 * Hkv * D);  // K and V interleaved per token, as the reference's buffers
  for (auto& x : q) x = to_half(0.5f * uniform() + (uniform() > 0 ? 0.01f : -0.01f));
  for (auto& x : kv) x = to_half(0.5f * uniform() + (uniform() > 0 ? 0.01f : -0.01f));

  void *dq, *dkv, *dmeta, *dout, *dlse;
  HIP_OK(hipMalloc(&dq, q.size() * 2));
  HIP_OK(hipMalloc(&dkv, kv.size() * 2));
  HIP_OK(hipMalloc(&dmeta, 6 * B * 4));
  HIP_OK(hipMalloc(&dout, (size_t)Tq * Hq * D * 4));
  HIP_OK(hipMalloc(&dlse, (size_t)Tq * Hq * 4));
  HIP_OK(hipMemcpy(dq, q.data(), q.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dkv, kv.data(), kv.size() * 2, hipMemcpyHostToDevice));
  int32_t meta[6 * B];
  memcpy(meta + 0 * B, q_start, sizeof q_start);
  memcpy(meta + 1 * B, q_len, sizeof q_len);
  memcpy(meta + 2 * B, q_first, sizeof q_first);
  memcpy(meta + 3 * B, kv_start, sizeof kv_start);
  memcpy(meta + 4 * B, kv_len, sizeof kv_len);
  memcpy(meta + 5 * B, kv_first, sizeof kv_first);
  HIP_OK(hipMemcpy(dmeta, meta, sizeof meta, hipMemcpyHostToDevice));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  lsattn_prefill_args a = {};
  a.q = dq;
  a.k = dkv;
  a.v = (const uint16_t*)dkv + (size_t)Hkv * D;
  a.q_stride_t = Hq * D;
  a.q_stride_h = D;
  a.k_stride_t = a.v_stride_t = 2 * Hkv * D;
  a.k_stride_h = a.v_stride_h = D;
  const int32_t* m = (const int32_t*)dmeta;
  a.q_b_start_loc = m;
  a.q_b_seq_len = m + B;
  a.q_first_token_global_idx = m + 2 * B;
  a.kv_b_start_loc = m + 3 * B;
  a.kv_b_seq_len = m + 4 * B;
  a.kv_first_token_global_idx = m + 5 * B;
  a.batch = B;
  a.num_q_heads = Hq;
  a.num_kv_heads = Hkv;
  a.head_dim = D;
  a.dtype = LSATTN_F16;
  a.sp_peers = P;
  a.max_q_len = 300;
  a.sm_scale = 1.0f / sqrtf((float)D);
  a.o = dout;
  a.o_stride_t = Hq * D;
  a.o_stride_h = D;
  a.o_dtype = LSATTN_F32;
  a.lse = (float*)dlse;

  // the reference on the host: key n of a chunk (global position kv_first + n P) counts for row m (q_first + m P) iff it
  // is not later
  std::vector<double> o_ref((size_t)Tq * Hq * D, 0.0), lse_ref((size_t)Tq * Hq, -INFINITY);
  for (int b = 0; b < B; b++)
    for (int r = 0; r < q_len[b]; r++)
      for (int h = 0; h < Hq; h++) {
        const int kh = h / (Hq / Hkv);
        const int64_t qpos = q_first[b] + (int64_t)r * P;
        const uint16_t* qrow = &q[((size_t)(q_start[b] + r) * Hq + h) * D];
        std::vector<double> s;
        double mx = -1e300;
        for (int n = 0; n < kv_len[b] && kv_first[b] + (int64_t)n * P <= qpos; n++) {
          const uint16_t* krow = &kv[((size_t)(kv_start[b] + n) * 2 * Hkv + kh) * D];
          double acc = 0;
          for (int d = 0; d < D; d++) acc += (double)from_half(qrow[d]) * from_half(krow[d]);
          s.push_back(acc / sqrt((double)D));
          mx = s.back() > mx ? s.back() : mx;
        }
        if (s.empty()) continue;  // a row that sees no key: O = 0, LSE = -inf
        double sum = 0;
        double* o = &o_ref[((size_t)(q_start[b] + r) * Hq + h) * D];
        for (size_t n = 0; n < s.size(); n++) {
          const double p = exp(s[n] - mx);
          sum += p;
          const uint16_t* vrow = &kv[((size_t)(kv_start[b] + n) * 2 * Hkv + Hkv + kh) * D];
          for (int d = 0; d < D; d++) o[d] += p * from_half(vrow[d]);
        }
        for (int d = 0; d < D; d++) o[d] /= sum;
        lse_ref[(size_t)(q_start[b] + r) * Hq + h] = mx + log(sum);
      }

  int bad = 0;
  for (int pass = 0; pass < 2; pass++) {
    const int rc = pass == 0 ? lsattn_prefill_step(&a, stream) : lsattn_prefill_step_accumulate(&a, stream);
    if (rc != LSATTN_OK) {
      fprintf(stderr, "entry point %d returned %d (%s)\n", pass, rc, lsattn_strerror(rc));
      return 3;
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> o((size_t)Tq * Hq * D), lse((size_t)Tq * Hq);
    HIP_OK(hipMemcpy(o.data(), dout, o.size() * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(lse.data(), dlse, lse.size() * 4, hipMemcpyDeviceToHost));
    double max_abs = 0, max_lse = 0;
    for (size_t j = 0; j < o.size(); j++) {
      const double e = fabs((double)o[j] - o_ref[j]);
      if (!(e <= 2e-3)) bad++;
      max_abs = e > max_abs ? e : max_abs;
    }
    for (size_t j = 0; j < lse.size(); j++) {
      const double want = lse_ref[j] + (pass == 1 ? log(2.0) : 0.0);
      if (std::isinf(want)) {
        if (!(std::isinf(lse[j]) && lse[j] < 0)) bad++;
        continue;
      }
      const double e = fabs((double)lse[j] - want) / (fabs(want) > 1 ? fabs(want) : 1);
      if (!(e <= 1e-4)) bad++;
      max_lse = e > max_lse ? e : max_lse;
    }
    printf("%s: max |O - ref| = %.3e (bar 2e-3), max rel LSE error = %.3e (bar 1e-4)\n",
           pass == 0 ? "lsattn_prefill_step" : "lsattn_prefill_step_accumulate", max_abs, max_lse);
  }
  printf(bad ? "FAILED: %d values outside the bars\n" : "ok\n", bad);
  return bad ? 1 : 0;
}
