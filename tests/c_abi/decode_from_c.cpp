// A consumer of the C ABI with no Python and no PyTorch in the process: HIP runtime calls for memory, include/lsattn.h for
// the attention.  Token-indexed flash decoding (stage 1 + stage 2 through lsattn_decode_attention, and the same through
// the entry point that allocates nothing) over a scattered pool, checked against a double-precision loop on the host.
// Built by loongserve_amd/build.py next to the library; run by tests/test_gpu_c_abi.py.  Exit status 0 = within the bars.
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

// float <-> IEEE half, round to nearest even (values here are small normals)
static uint16_t to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  int32_t exp = (int32_t)((x >> 23) & 0xff) - 127 + 15;
  uint32_t man = x & 0x7fffffu;
  if (exp <= 0) return (uint16_t)sign;  // flush: not produced by the generator below
  if (exp >= 31) return (uint16_t)(sign | 0x7c00u);
  uint32_t h = sign | ((uint32_t)exp << 10) | (man >> 13);
  const uint32_t rest = man & 0x1fffu;
  if (rest > 0x1000u || (rest == 0x1000u && (h & 1))) h++;
  return (uint16_t)h;
}
static float from_half(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu;
  uint32_t x;
  if (exp == 0) x = sign;  // zero (no subnormals generated)
  else x = sign | ((exp - 15 + 127) << 23) | (man << 13);
  float f;
  memcpy(&f, &x, 4);
  return f;
}
static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static float uniform() {  // xorshift64*, in [-1, 1)
  rng_state ^= rng_state >> 12;
  rng_state ^= rng_state << 25;
  rng_state ^= rng_state >> 27;
  return (float)((double)((rng_state * 0x2545F4914F6CDD1Dull) >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}

int main(int argc, char** argv) {
  const int Hq = argc > 1 ? atoi(argv[1]) : 32, Hkv = argc > 2 ? atoi(argv[2]) : 8, D = 128, BS = 256;
  const int B = 3;
  const int lens[B] = {5000, 1, 777};
  const int max_len = 5000, max_seq = max_len + 3, max_req = B + 1, slots = 7000;
  const int req_idx[B] = {2, 0, 3};
  const int nblk = (max_len + BS - 1) / BS;
  std::vector<uint16_t> q((size_t)B * Hq * D), kv((size_t)slots * 2 * Hkv * D);
  for (auto& x : q) x = to_half(0.5f * uniform() + (uniform() > 0 ? 0.01f : -0.01f));
  for (auto& x : kv) x = to_half(0.5f * uniform() + (uniform() > 0 ? 0.01f : -0.01f));
  // every token of every request in a slot of its own, scattered: slot = (a * i + c) mod slots with a coprime to slots
  std::vector<int32_t> table((size_t)max_req * max_seq, 2147483647);
  int64_t i = 0;
  for (int b = 0; b < B; b++)
    for (int t = 0; t < lens[b]; t++, i++) table[(size_t)req_idx[b] * max_seq + t] = (int32_t)((i * 4099 + 17) % slots);

  void *dq, *dkv, *dtab, *dreq, *dlen, *dmo, *dml, *dout, *dlse;
  HIP_OK(hipMalloc(&dq, q.size() * 2));
  HIP_OK(hipMalloc(&dkv, kv.size() * 2));
  HIP_OK(hipMalloc(&dtab, table.size() * 4));
  HIP_OK(hipMalloc(&dreq, B * 4));
  HIP_OK(hipMalloc(&dlen, B * 4));
  HIP_OK(hipMalloc(&dmo, (size_t)nblk * B * Hq * D * 4));
  HIP_OK(hipMalloc(&dml, (size_t)nblk * B * Hq * 4));
  HIP_OK(hipMalloc(&dout, (size_t)B * Hq * D * 4));
  HIP_OK(hipMalloc(&dlse, (size_t)B * Hq * 4));
  HIP_OK(hipMemcpy(dq, q.data(), q.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dkv, kv.data(), kv.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dtab, table.data(), table.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dreq, req_idx, B * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dlen, lens, B * 4, hipMemcpyHostToDevice));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  lsattn_decode_stage1_args s1 = {};
  s1.mid_o = (float*)dmo;
  s1.mid_o_logexpsum = (float*)dml;
  s1.q = dq;
  s1.k = dkv;                                       // K rows are heads 0 .. Hkv-1 of a pool row, V rows the other half
  s1.v = (const uint16_t*)dkv + (size_t)Hkv * D;
  s1.k_stride_0 = s1.v_stride_0 = 2 * Hkv * D;
  s1.k_stride_1 = s1.v_stride_1 = D;
  s1.sm_scale = 1.0f / sqrtf((float)D);
  s1.dtype = LSATTN_F16;
  s1.req_to_tokens = (const int32_t*)dtab;
  s1.b_req_idx = (const int32_t*)dreq;
  s1.b_seqlen = (const int32_t*)dlen;
  s1.batch = B;
  s1.num_q_heads = Hq;
  s1.num_kv_heads = Hkv;
  s1.num_blocks = nblk;
  s1.head_dim = D;
  s1.max_seq_len = max_seq;
  s1.seq_block_size = BS;
  s1.max_len_in_batch = max_len;
  lsattn_decode_stage2_args s2 = {};
  s2.o = dout;
  s2.o_dtype = LSATTN_F32;
  s2.out_logexpsum = (float*)dlse;
  s2.b_seqlen = (const int32_t*)dlen;
  s2.mid_o = (const float*)dmo;
  s2.mid_o_logexpsum = (const float*)dml;
  s2.batch = B;
  s2.num_heads = Hq;
  s2.num_seq_blocks = nblk;
  s2.head_dim = D;
  s2.block_seq = BS;

  // the reference on the host, in double
  std::vector<double> o_ref((size_t)B * Hq * D), lse_ref((size_t)B * Hq);
  const int group = Hq / Hkv;
  for (int b = 0; b < B; b++)
    for (int h = 0; h < Hq; h++) {
      const int kh = h / group;
      std::vector<double> s(lens[b]);
      double mx = -1e300;
      for (int t = 0; t < lens[b]; t++) {
        const size_t row = (size_t)table[(size_t)req_idx[b] * max_seq + t] * 2 * Hkv * D + (size_t)kh * D;
        double acc = 0;
        for (int d = 0; d < D; d++) acc += (double)from_half(q[((size_t)b * Hq + h) * D + d]) * from_half(kv[row + d]);
        s[t] = acc / sqrt((double)D);
        mx = s[t] > mx ? s[t] : mx;
      }
      double sum = 0;
      std::vector<double> o(D, 0.0);
      for (int t = 0; t < lens[b]; t++) {
        const double p = exp(s[t] - mx);
        sum += p;
        const size_t row = (size_t)table[(size_t)req_idx[b] * max_seq + t] * 2 * Hkv * D + (size_t)(Hkv + kh) * D;
        for (int d = 0; d < D; d++) o[d] += p * from_half(kv[row + d]);
      }
      for (int d = 0; d < D; d++) o_ref[((size_t)b * Hq + h) * D + d] = o[d] / sum;
      lse_ref[(size_t)b * Hq + h] = mx + log(sum);
    }

  int bad = 0;
  for (int pass = 0; pass < 3; pass++) {
    HIP_OK(hipMemsetAsync(dout, 0xff, (size_t)B * Hq * D * 4, stream));
    HIP_OK(hipMemsetAsync(dlse, 0xff, (size_t)B * Hq * 4, stream));
    int rc;
    if (pass == 0) {
      rc = lsattn_decode_attention(&s1, &s2, stream);
    } else if (pass == 2) {
      // the same buffers with a request's partials side by side ([batch, blocks, heads, head_dim])
      lsattn_decode_stage1_args t1 = s1;
      lsattn_decode_stage2_args t2 = s2;
      t1.partials_by_request = t2.partials_by_request = 1;
      rc = lsattn_decode_attention(&t1, &t2, stream);
    } else {
      // the entry point that allocates nothing keeps the partials in the library: the caller names none
      lsattn_decode_stage1_args t1 = s1;
      lsattn_decode_stage2_args t2 = s2;
      t1.mid_o = t1.mid_o_logexpsum = nullptr;
      t2.mid_o = t2.mid_o_logexpsum = nullptr;
      rc = lsattn_decode_attention_static(&t1, &t2, stream);
    }
    if (rc != LSATTN_OK) {
      fprintf(stderr, "entry point %d returned %d (%s)\n", pass, rc, lsattn_strerror(rc));
      return 3;
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> o((size_t)B * Hq * D), lse((size_t)B * Hq);
    HIP_OK(hipMemcpy(o.data(), dout, o.size() * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(lse.data(), dlse, lse.size() * 4, hipMemcpyDeviceToHost));
    double max_abs = 0, max_lse = 0;
    for (size_t j = 0; j < o.size(); j++) {
      const double e = fabs((double)o[j] - o_ref[j]);
      if (!(e <= 2e-3)) bad++;  // (also catches NaN)
      max_abs = e > max_abs ? e : max_abs;
    }
    for (size_t j = 0; j < lse.size(); j++) {
      const double e = fabs((double)lse[j] - lse_ref[j]) / (fabs(lse_ref[j]) > 1 ? fabs(lse_ref[j]) : 1);
      if (!(e <= 1e-4)) bad++;
      max_lse = e > max_lse ? e : max_lse;
    }
    printf("%s: heads %d/%d, max |O - ref| = %.3e (bar 2e-3), max rel LSE error = %.3e (bar 1e-4)\n",
           pass == 0 ? "lsattn_decode_attention" : pass == 1 ? "lsattn_decode_attention_static" : "lsattn_decode_attention, partials by request", Hq, Hkv,
           max_abs, max_lse);
  }
  printf(bad ? "FAILED: %d values outside the bars\n" : "ok\n", bad);
  return bad ? 1 : 0;
}
