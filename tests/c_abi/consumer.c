/*
 * A consumer of the C ABI written in plain C, with nothing but the HIP runtime beside it: device buffers from
 * hipMalloc, the library's entry points, and the expected values computed right here in double precision from the
 * definitions (log-softmax, entropy, the supervised loss and its gradient; for the lm_head entry points the product
 * hidden @ weight.T as well).  Exit status 0 = every check passed.
 *
 * Build (done by __graft_entry__.build()):
 *   gcc -std=c99 -D__HIP_PLATFORM_AMD__ -I/opt/rocm/include -Iinclude tests/c_abi/consumer.c \
 *       -o tests/c_abi/consumer -Lareal_amd -lareal_amd -L/opt/rocm/lib -lamdhip64 -lm -Wl,-rpath,...
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "areal_amd.h"

#define T 7
#define V 1003
/* lm_head part: hidden [LT, LH] and weight [LV, LH] in bf16 */
#define LT 40
#define LH 64
#define LV 520

#define HIP_OK(call)                                                                 \
  do {                                                                               \
    hipError_t e_ = (call);                                                          \
    if (e_ != hipSuccess) {                                                          \
      fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));              \
      return 2;                                                                      \
    }                                                                                \
  } while (0)

#define AA_CHECK(call)                                                               \
  do {                                                                               \
    int s_ = (call);                                                                 \
    if (s_ != AA_OK) {                                                               \
      fprintf(stderr, "%s failed: %s\n", #call, aa_status_string(s_));               \
      return 3;                                                                      \
    }                                                                                \
  } while (0)

static int close_to(double got, double want, double tol, const char* what, int t) {
  if (fabs(got - want) <= tol * (1.0 + fabs(want))) return 1;
  fprintf(stderr, "%s[%d]: got %.9g, expected %.9g\n", what, t, got, want);
  return 0;
}

int main(void) {
  static float logits[T * V];
  int64_t labels[T];
  uint8_t mask[T] = {0, 1, 1, 0, 1, 1, 1};
  const float inv_temperature = 1.0f / 0.8f;
  uint32_t state = 12345u;
  for (int i = 0; i < T * V; ++i) {  /* a small linear congruential generator: values in [-4, 4) */
    state = state * 1664525u + 1013904223u;
    logits[i] = (float)(state >> 8) / (float)(1u << 24) * 8.0f - 4.0f;
  }
  for (int t = 0; t < T; ++t) labels[t] = (t * 131 + 7) % V;

  /* expected values from the definitions, in double */
  double want_logp[T], want_entropy[T];
  int n_valid = 0;
  for (int t = 0; t < T; ++t) {
    double mx = -1e300, s = 0.0, u = 0.0;
    for (int j = 0; j < V; ++j) mx = fmax(mx, (double)logits[t * V + j] * inv_temperature);
    for (int j = 0; j < V; ++j) {
      const double z = (double)logits[t * V + j] * inv_temperature;
      s += exp(z - mx);
      u += exp(z - mx) * z;
    }
    const double lse = mx + log(s);
    want_logp[t] = (double)logits[t * V + labels[t]] * inv_temperature - lse;
    want_entropy[t] = lse - u / s;
    n_valid += mask[t] ? 1 : 0;
  }
  double want_loss = 0.0;
  for (int t = 0; t < T; ++t) want_loss -= mask[t] ? want_logp[t] : 0.0;
  want_loss /= (double)n_valid + 1e-5;

  float *d_logits, *d_logp, *d_entropy, *d_loss, *d_g, *d_stat, *d_ppl;
  int64_t* d_labels;
  uint8_t* d_mask;
  int32_t *d_count, *d_cu, *d_seq_count;
  double* d_seq_logp;
  const int32_t cu[3] = {0, 3, T};
  HIP_OK(hipMalloc((void**)&d_logits, sizeof(logits)));
  HIP_OK(hipMalloc((void**)&d_labels, sizeof(labels)));
  HIP_OK(hipMalloc((void**)&d_mask, 256));
  HIP_OK(hipMalloc((void**)&d_logp, T * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_entropy, T * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_g, T * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_stat, T * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_loss, 256));
  HIP_OK(hipMalloc((void**)&d_ppl, 256));
  HIP_OK(hipMalloc((void**)&d_count, 256));
  HIP_OK(hipMalloc((void**)&d_cu, 256));
  HIP_OK(hipMalloc((void**)&d_seq_count, 256));
  HIP_OK(hipMalloc((void**)&d_seq_logp, 256));
  HIP_OK(hipMemcpy(d_logits, logits, sizeof(logits), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_labels, labels, sizeof(labels), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_mask, mask, sizeof(mask), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_cu, cu, sizeof(cu), hipMemcpyHostToDevice));

  if (aa_version() < 100) return 4;
  /* the log-prob op, the token count, the supervised loss on the log-probs: all on the default stream */
  AA_CHECK(aa_logits_fwd(d_logits, AA_F32, T, V, V, d_labels, inv_temperature, d_logp, d_entropy, NULL, NULL, NULL,
                         NULL, NULL));
  AA_CHECK(aa_count_nonzero_u8(d_mask, T, d_count, NULL));
  AA_CHECK(aa_sft_loss(d_logp, d_mask, T, d_cu, 2, d_count, NULL, d_loss, d_g, d_stat, d_seq_logp, d_seq_count, d_ppl,
                       NULL));
  HIP_OK(hipDeviceSynchronize());

  float logp[T], entropy[T], g[T], loss, ppl[2];
  int32_t count, seq_count[3];
  double seq_logp[3];
  HIP_OK(hipMemcpy(logp, d_logp, sizeof(logp), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(entropy, d_entropy, sizeof(entropy), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(g, d_g, sizeof(g), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(&loss, d_loss, sizeof(loss), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(&count, d_count, sizeof(count), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(ppl, d_ppl, sizeof(ppl), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(seq_count, d_seq_count, sizeof(seq_count), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(seq_logp, d_seq_logp, sizeof(seq_logp), hipMemcpyDeviceToHost));

  int ok = count == n_valid;
  for (int t = 0; t < T; ++t) {
    ok &= close_to(logp[t], want_logp[t], 2e-6, "logp", t);
    ok &= close_to(entropy[t], want_entropy[t], 2e-6, "entropy", t);
    ok &= close_to(g[t], mask[t] ? -1.0 / ((double)n_valid + 1e-5) : 0.0, 1e-6, "g_logp", t);
  }
  ok &= close_to(loss, want_loss, 2e-6, "loss", 0);
  /* sequence 0 = tokens 0..2 (two selected), sequence 1 = tokens 3..6 (three selected) */
  ok &= seq_count[0] == 2 && seq_count[1] == 3 && seq_count[2] == 0;
  ok &= close_to(seq_logp[0], (want_logp[1] + want_logp[2]) / 2.0, 2e-6, "seq_logp", 0);
  ok &= close_to(seq_logp[1], (want_logp[4] + want_logp[5] + want_logp[6]) / 3.0, 2e-6, "seq_logp", 1);
  ok &= close_to(ppl[0], exp(-(want_logp[1] + want_logp[2]) / 2.0), 1e-5, "ppl", 0);

  /* a bad argument is refused before anything is queued */
  ok &= aa_logits_fwd(d_logits, AA_F32, T, V, V, d_labels, 0.0f, d_logp, NULL, NULL, NULL, NULL, NULL, NULL) ==
        AA_ERR_INVALID_ARGUMENT;

  /* lm_head: log-prob and entropy of softmax(hidden @ weight.T / temperature) without the logits in memory, through
   * aa_lmhead_fwd (workspace from the caller) and aa_lmhead_fwd_static (no workspace, nothing allocated).  The bf16
   * inputs are small multiples of 1/64 (hidden) and 1/256 (weight), exact in bf16, so the products are exact. */
  {
    static uint16_t hid[LT * LH], wgt[LV * LH];
    static double hid_d[LT * LH], wgt_d[LV * LH];
    int64_t llabels[LT];
    for (int i = 0; i < LT * LH + LV * LH; ++i) {
      state = state * 1664525u + 1013904223u;
      const int k = (int)((state >> 8) % 255u) - 127; /* -127 .. 127 */
      const int is_w = i >= LT * LH;
      const float f = (float)k / (is_w ? 256.0f : 64.0f); /* weights a quarter of the hidden states' range */
      uint32_t bits;
      memcpy(&bits, &f, 4);
      if (is_w) { wgt[i - LT * LH] = (uint16_t)(bits >> 16); wgt_d[i - LT * LH] = f; }
      else { hid[i] = (uint16_t)(bits >> 16); hid_d[i] = f; }
    }
    double want_lp[LT], want_ent[LT], want_max[LT], want_min[LT];
    for (int t = 0; t < LT; ++t) {
      static double z[LV];
      double mx = -1e300, sum = 0.0, u = 0.0;
      llabels[t] = (t * 37 + 11) % LV;
      for (int v = 0; v < LV; ++v) {
        double acc = 0.0;
        for (int h = 0; h < LH; ++h) acc += hid_d[t * LH + h] * wgt_d[v * LH + h];
        z[v] = acc * inv_temperature;
        mx = fmax(mx, z[v]);
        want_max[t] = v == 0 ? acc : fmax(want_max[t], acc); /* extrema of the raw logits */
        want_min[t] = v == 0 ? acc : fmin(want_min[t], acc);
      }
      for (int v = 0; v < LV; ++v) { sum += exp(z[v] - mx); u += exp(z[v] - mx) * z[v]; }
      want_lp[t] = z[llabels[t]] - (mx + log(sum));
      want_ent[t] = (mx + log(sum)) - u / sum;
    }
    uint16_t *d_hid, *d_wgt;
    int64_t* d_ll;
    float *d_lp, *d_ent, *d_lp2, *d_ent2, *d_vmax, *d_vmin;
    void* d_ws;
    const int64_t ws_bytes = aa_lmhead_fwd_stats_workspace_bytes(LT, LH, LV); /* with the extrema of the logits */
    if (ws_bytes <= 0) return 5;
    HIP_OK(hipMalloc((void**)&d_hid, sizeof(hid)));
    HIP_OK(hipMalloc((void**)&d_wgt, sizeof(wgt)));
    HIP_OK(hipMalloc((void**)&d_ll, sizeof(llabels)));
    HIP_OK(hipMalloc((void**)&d_lp, LT * sizeof(float)));
    HIP_OK(hipMalloc((void**)&d_ent, LT * sizeof(float)));
    HIP_OK(hipMalloc((void**)&d_lp2, LT * sizeof(float)));
    HIP_OK(hipMalloc((void**)&d_ent2, LT * sizeof(float)));
    HIP_OK(hipMalloc((void**)&d_vmax, LT * sizeof(float)));
    HIP_OK(hipMalloc((void**)&d_vmin, LT * sizeof(float)));
    HIP_OK(hipMalloc(&d_ws, (size_t)ws_bytes));
    HIP_OK(hipMemcpy(d_hid, hid, sizeof(hid), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_wgt, wgt, sizeof(wgt), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_ll, llabels, sizeof(llabels), hipMemcpyHostToDevice));
    AA_CHECK(aa_lmhead_prepare());
    AA_CHECK(aa_lmhead_fwd(d_hid, d_wgt, LT, LH, LV, d_ll, inv_temperature, d_lp, d_ent, NULL, NULL, d_vmax, d_vmin, d_ws, ws_bytes,
                           NULL));
    AA_CHECK(aa_lmhead_fwd_static(d_hid, d_wgt, LT, LH, LV, d_ll, inv_temperature, d_lp2, d_ent2, NULL, NULL, NULL));
    HIP_OK(hipDeviceSynchronize());
    float lp[LT], ent[LT], lp2[LT], ent2[LT], vmax[LT], vmin[LT];
    HIP_OK(hipMemcpy(vmax, d_vmax, sizeof(vmax), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(vmin, d_vmin, sizeof(vmin), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(lp, d_lp, sizeof(lp), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(ent, d_ent, sizeof(ent), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(lp2, d_lp2, sizeof(lp2), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(ent2, d_ent2, sizeof(ent2), hipMemcpyDeviceToHost));
    for (int t = 0; t < LT; ++t) {
      ok &= close_to(lp[t], want_lp[t], 5e-6, "lm_head logp", t);
      ok &= close_to(ent[t], want_ent[t], 5e-6, "lm_head entropy", t);
      ok &= close_to(vmax[t], want_max[t], 5e-6, "lm_head vocab max", t);
      ok &= close_to(vmin[t], want_min[t], 5e-6, "lm_head vocab min", t);
      ok &= lp[t] == lp2[t] && ent[t] == ent2[t]; /* the two entry points run the same kernels */
    }
    /* H must be a multiple of 8 */
    ok &= aa_lmhead_fwd(d_hid, d_wgt, LT, LH - 4, LV, d_ll, inv_temperature, d_lp, d_ent, NULL, NULL, NULL, NULL, d_ws, ws_bytes, NULL) ==
          AA_ERR_UNSUPPORTED;
    hipFree(d_hid); hipFree(d_wgt); hipFree(d_ll); hipFree(d_lp); hipFree(d_ent); hipFree(d_lp2); hipFree(d_ent2);
    hipFree(d_vmax); hipFree(d_vmin); hipFree(d_ws);
  }

  hipFree(d_logits); hipFree(d_labels); hipFree(d_mask); hipFree(d_logp); hipFree(d_entropy); hipFree(d_g);
  hipFree(d_stat); hipFree(d_loss); hipFree(d_ppl); hipFree(d_count); hipFree(d_cu); hipFree(d_seq_count);
  hipFree(d_seq_logp);
  if (!ok) return 1;
  printf("c_abi consumer ok: %d tokens, loss %.6f\n", T, loss);
  return 0;
}
