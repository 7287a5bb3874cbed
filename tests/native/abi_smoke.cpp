// A host program with no Python and no torch in it: it links libomnikv_hip.so, feeds it
// device buffers it allocated itself through the HIP runtime, and checks every result against
// plain loops over the same bf16 values.  It exists to show that the C ABI is the whole
// boundary: what a C, C++, Go (cgo) or Java (JNI) host would bind is exactly what is called here.
//
//   filter layer   okv_dense_attn with the score side output (softmax per head, summed over heads)
//   selection      okv_topk on those scores  -> must equal a stable sort of the SAME device scores
//   sparse layer   okv_sparse_attn over the selected rows + one tail row
//   bookkeeping    okv_workspace_bytes, okv_gather_rows, error reporting for a bad argument
//   no allocation  okv_sparse_attn_noalloc must reproduce okv_sparse_attn bit for bit
//   host tier      okv_offload_plan + okv_offload_fetch over two overlapping selections: the staged
//                  rows are exactly the second selection, and only its new rows were copied
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>

#include "../../include/omnikv_hip.h"

#define HIP_OK(e)                                                                      \
  do {                                                                                 \
    hipError_t err_ = (e);                                                             \
    if (err_ != hipSuccess) {                                                          \
      std::fprintf(stderr, "%s: %s (line %d)\n", #e, hipGetErrorString(err_), __LINE__); \
      return 2;                                                                        \
    }                                                                                  \
  } while (0)
#define OKV(e)                                                                                  \
  do {                                                                                          \
    int rc_ = (e);                                                                              \
    if (rc_ != OKV_OK) {                                                                        \
      std::fprintf(stderr, "%s -> %d %s: %s (line %d)\n", #e, rc_, okv_strerror(rc_), okv_last_error(), \
                   __LINE__);                                                                   \
      return 3;                                                                                 \
    }                                                                                           \
  } while (0)

static uint16_t to_bf16(float f) {  // round to nearest even
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

struct Lcg {  // deterministic values in (-1, 1)
  uint64_t s;
  float next() {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return (float)((int64_t)(s >> 33) - (1ll << 30)) / (float)(1ll << 30);
  }
};

int main() {
  const int N = 3000, T = 1, HQ = 32, HKV = 8, D = 128, G = HQ / HKV, K_SEL = 201;
  const float scale = 1.0f / std::sqrt((float)D);
  int ndev = 0;
  HIP_OK(hipGetDeviceCount(&ndev));
  if (ndev < 1) {
    std::fprintf(stderr, "no GPU\n");
    return 2;
  }
  if (okv_version() < 1) return 4;

  // ---- host data: K, V as (Hkv, N+T, D) bf16, q as (Hq, D)
  Lcg rng{12345};
  const size_t rows = (size_t)N + T;
  std::vector<uint16_t> hk(HKV * rows * D), hv(HKV * rows * D), hq(HQ * D);
  for (auto& x : hk) x = to_bf16(rng.next() * 2.0f);
  for (auto& x : hv) x = to_bf16(rng.next());
  for (auto& x : hq) x = to_bf16(rng.next() * 3.0f);
  auto Kf = [&](int g, int t, int d) { return from_bf16(hk[((size_t)g * rows + t) * D + d]); };
  auto Vf = [&](int g, int t, int d) { return from_bf16(hv[((size_t)g * rows + t) * D + d]); };
  auto Qf = [&](int h, int d) { return from_bf16(hq[(size_t)h * D + d]); };

  void *dk, *dv, *dq, *dout, *dws, *dgather;
  float* dscores;
  int32_t* didx;
  HIP_OK(hipMalloc(&dk, hk.size() * 2));
  HIP_OK(hipMalloc(&dv, hv.size() * 2));
  HIP_OK(hipMalloc(&dq, hq.size() * 2));
  HIP_OK(hipMalloc(&dout, (size_t)HQ * D * 2));
  HIP_OK(hipMalloc((void**)&dscores, (size_t)N * 4));
  HIP_OK(hipMalloc((void**)&didx, (size_t)K_SEL * 4));
  HIP_OK(hipMalloc(&dgather, (size_t)HKV * K_SEL * D * 2));
  HIP_OK(hipMemcpy(dk, hk.data(), hk.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dv, hv.data(), hv.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dq, hq.data(), hq.size() * 2, hipMemcpyHostToDevice));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  okv_kv_layout_t lay;
  std::memset(&lay, 0, sizeof(lay));
  lay.dtype = OKV_BF16;
  lay.num_q_heads = HQ;
  lay.num_kv_heads = HKV;
  lay.head_dim = D;
  lay.token_stride = D;
  lay.head_stride = (int64_t)rows * D;
  lay.batch_stride = (int64_t)HKV * rows * D;

  // ---- one workspace for all calls: the largest any of them asks for
  size_t ws_bytes = 0;
  for (int op : {OKV_OP_DENSE_ATTN, OKV_OP_TOPK, OKV_OP_SPARSE_ATTN, OKV_OP_DENSE_ATTN_SELECT, OKV_OP_DENSE_ATTN_WINDOW}) {
    okv_shape_t sh;
    std::memset(&sh, 0, sizeof(sh));
    sh.batch = 1;
    sh.num_q_heads = HQ;
    sh.num_kv_heads = HKV;
    sh.head_dim = D;
    sh.max_seq_len = N + T;
    sh.max_tail_len = T;
    sh.with_scores = 1;
    size_t b = 0;
    OKV(okv_workspace_bytes(op, &sh, &b));
    ws_bytes = std::max(ws_bytes, b);
  }
  HIP_OK(hipMalloc(&dws, ws_bytes));

  // ---- a bad call is refused with a message, nothing is launched
  if (okv_topk(nullptr, N, nullptr, N, nullptr, K_SEL, 1, didx, K_SEL, dws, ws_bytes, stream) != OKV_ERR_INVALID ||
      std::strlen(okv_last_error()) == 0) {
    std::fprintf(stderr, "NULL scores were not refused\n");
    return 5;
  }

  // ---- filter layer: attention over all N+T rows, scores over the first N
  OKV(okv_dense_attn(dq, dk, dv, &lay, nullptr, N + T, 1, scale, dout, nullptr, N, OKV_REDUCE_SUM,
                     OKV_NORM_SOFTMAX, dscores, N, dws, ws_bytes, stream));
  OKV(okv_topk(dscores, N, nullptr, N, nullptr, K_SEL, 1, didx, K_SEL, dws, ws_bytes, stream));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<float> scores(N);
  std::vector<int32_t> idx(K_SEL);
  std::vector<uint16_t> out(HQ * D);
  HIP_OK(hipMemcpy(scores.data(), dscores, (size_t)N * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(idx.data(), didx, (size_t)K_SEL * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(out.data(), dout, out.size() * 2, hipMemcpyDeviceToHost));

  // host reference: logits in double
  std::vector<double> logit((size_t)HQ * rows);
  for (int h = 0; h < HQ; ++h)
    for (size_t t = 0; t < rows; ++t) {
      double s = 0;
      for (int d = 0; d < D; ++d) s += (double)Qf(h, d) * Kf(h / G, (int)t, d);
      logit[h * rows + t] = s * scale;
    }
  // scores: softmax over the first N rows per head, summed over heads
  std::vector<double> want_scores(N, 0.0);
  for (int h = 0; h < HQ; ++h) {
    double m = -1e300, z = 0;
    for (int t = 0; t < N; ++t) m = std::max(m, logit[h * rows + t]);
    for (int t = 0; t < N; ++t) z += std::exp(logit[h * rows + t] - m);
    for (int t = 0; t < N; ++t) want_scores[t] += std::exp(logit[h * rows + t] - m) / z;
  }
  double worst = 0;
  for (int t = 0; t < N; ++t)
    worst = std::max(worst, std::fabs(scores[t] - want_scores[t]) / (std::fabs(want_scores[t]) + 1e-6));
  if (worst > 1e-3) {
    std::fprintf(stderr, "scores differ: relative error %g\n", worst);
    return 6;
  }
  // selection: a stable sort of the device's own scores, bit for bit
  std::vector<int32_t> order(N);
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return scores[a] > scores[b]; });
  std::vector<int32_t> want_idx(order.begin(), order.begin() + K_SEL);
  std::sort(want_idx.begin(), want_idx.end());
  if (want_idx != idx) {
    std::fprintf(stderr, "top-k indices differ from the stable sort of the same scores\n");
    return 7;
  }
  // attention over row set `sel` for head h, in double
  auto attend = [&](const std::vector<int>& sel, int h, std::vector<double>& o) {
    double m = -1e300, z = 0;
    for (int t : sel) m = std::max(m, logit[h * rows + t]);
    o.assign(D, 0.0);
    for (int t : sel) {
      const double p = std::exp(logit[h * rows + t] - m);
      z += p;
      for (int d = 0; d < D; ++d) o[d] += p * Vf(h / G, t, d);
    }
    for (int d = 0; d < D; ++d) o[d] /= z;
  };
  auto check_out = [&](const std::vector<int>& sel, const char* what) -> double {
    double w = 0;
    std::vector<double> o;
    for (int h = 0; h < HQ; ++h) {
      attend(sel, h, o);
      for (int d = 0; d < D; ++d) w = std::max(w, std::fabs(from_bf16(out[h * D + d]) - o[d]));
    }
    std::printf("%s: max abs error %.3g\n", what, w);
    return w;
  };
  std::vector<int> all(rows);
  std::iota(all.begin(), all.end(), 0);
  if (check_out(all, "dense attention") > 2e-2) return 8;

  // ---- the filter layer as one call: the same three outputs, bit for bit
  {
    void* dout2;
    float* dscores2;
    int32_t* didx2;
    HIP_OK(hipMalloc(&dout2, (size_t)HQ * D * 2));
    HIP_OK(hipMalloc((void**)&dscores2, (size_t)N * 4));
    HIP_OK(hipMalloc((void**)&didx2, (size_t)K_SEL * 4));
    OKV(okv_dense_attn_select(dq, dk, dv, &lay, nullptr, N + T, 1, scale, dout2, nullptr, N, OKV_REDUCE_SUM,
                              OKV_NORM_SOFTMAX, dscores2, N, nullptr, K_SEL, didx2, K_SEL, dws, ws_bytes, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> scores2(N);
    std::vector<int32_t> idx2(K_SEL);
    std::vector<uint16_t> out2(HQ * D);
    HIP_OK(hipMemcpy(scores2.data(), dscores2, (size_t)N * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(idx2.data(), didx2, (size_t)K_SEL * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(out2.data(), dout2, out2.size() * 2, hipMemcpyDeviceToHost));
    if (std::memcmp(scores2.data(), scores.data(), (size_t)N * 4) != 0 || idx2 != idx || out2 != out) {
      std::fprintf(stderr, "okv_dense_attn_select differs from okv_dense_attn + okv_topk\n");
      return 12;
    }
    // ---- a window selector with a window of one position (the current query): per token the
    // largest softmax probability over the heads; the attention is the same as above
    OKV(okv_dense_attn_window(dq, dq, (int64_t)HQ * D, D, D, 1, 0, dk, dv, &lay, nullptr, N + T, 1, scale, dout2,
                              nullptr, N, dscores2, N, dws, ws_bytes, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(scores2.data(), dscores2, (size_t)N * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(out2.data(), dout2, out2.size() * 2, hipMemcpyDeviceToHost));
    std::vector<double> want_w(N, 0.0);
    for (int h = 0; h < HQ; ++h) {
      double m = -1e300, z = 0;
      for (int t = 0; t < N; ++t) m = std::max(m, logit[h * rows + t]);
      for (int t = 0; t < N; ++t) z += std::exp(logit[h * rows + t] - m);
      for (int t = 0; t < N; ++t) want_w[t] = std::max(want_w[t], std::exp(logit[h * rows + t] - m) / z);
    }
    double ww = 0, wo = 0;
    for (int t = 0; t < N; ++t) ww = std::max(ww, std::fabs(scores2[t] - want_w[t]) / (std::fabs(want_w[t]) + 1e-6));
    for (int i = 0; i < HQ * D; ++i) wo = std::max(wo, (double)std::fabs(from_bf16(out2[i]) - from_bf16(out[i])));
    std::printf("window filter layer: scores relative error %.3g, attention vs the dense call %.3g\n", ww, wo);
    if (ww > 1e-3 || wo > 2e-2) return 13;
    HIP_OK(hipFree(dout2));
    HIP_OK(hipFree(dscores2));
    HIP_OK(hipFree(didx2));
  }

  // ---- sparse layer: the selected rows + the tail row (row N of the same buffers)
  const uint16_t* tk = (const uint16_t*)dk + (size_t)N * D;
  const uint16_t* tv = (const uint16_t*)dv + (size_t)N * D;
  OKV(okv_sparse_attn(dq, dk, dv, &lay, didx, K_SEL, nullptr, K_SEL, tk, tv, D, (int64_t)rows * D,
                      (int64_t)HKV * rows * D, nullptr, T, 1, scale, dout, dws, ws_bytes, stream));
  OKV(okv_gather_rows(dk, &lay, didx, K_SEL, nullptr, K_SEL, 1, dgather, D, (int64_t)K_SEL * D,
                      (int64_t)HKV * K_SEL * D, stream));
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(out.data(), dout, out.size() * 2, hipMemcpyDeviceToHost));
  std::vector<int> sel(idx.begin(), idx.end());
  sel.push_back(N);
  if (check_out(sel, "sparse attention") > 2e-2) return 9;
  std::vector<uint16_t> gathered((size_t)HKV * K_SEL * D);
  HIP_OK(hipMemcpy(gathered.data(), dgather, gathered.size() * 2, hipMemcpyDeviceToHost));
  for (int g = 0; g < HKV; ++g)
    for (int j = 0; j < K_SEL; ++j)
      if (std::memcmp(&gathered[((size_t)g * K_SEL + j) * D], &hk[((size_t)g * rows + idx[j]) * D], D * 2) != 0) {
        std::fprintf(stderr, "gathered row %d of head %d differs from its source\n", j, g);
        return 10;
      }

  // ---- the same sparse layer without a workspace: the library's fixed scratch, same bits
  {
    void* dout2;
    HIP_OK(hipMalloc(&dout2, (size_t)HQ * D * 2));
    OKV(okv_sparse_attn_noalloc(dq, dk, dv, &lay, didx, K_SEL, nullptr, K_SEL, tk, tv, D, (int64_t)rows * D,
                                (int64_t)HKV * rows * D, nullptr, T, 1, scale, dout2, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<uint16_t> out2(HQ * D);
    HIP_OK(hipMemcpy(out2.data(), dout2, out2.size() * 2, hipMemcpyDeviceToHost));
    if (out2 != out) {
      std::fprintf(stderr, "okv_sparse_attn_noalloc differs from okv_sparse_attn\n");
      return 11;
    }
    HIP_OK(hipFree(dout2));
  }

  // ---- incremental staging: rows of (N, 2, Hkv, D) = one 4 KB row per token (here in device memory; the
  // tier keeps them in pinned host memory), two selections that share every other token
  {
    const int KS = 64;
    const int64_t row_bytes = 2 * HKV * D * 2;
    std::vector<uint16_t> hsrc((size_t)N * row_bytes / 2);
    for (size_t i = 0; i < hsrc.size(); ++i) hsrc[i] = (uint16_t)(i * 2654435761u >> 16);
    std::vector<int32_t> sel_a(KS), sel_b(KS), minus(KS, -1), minus_n(N, -1);
    for (int j = 0; j < KS; ++j) sel_a[j] = 7 + 31 * j;                       // ascending, distinct
    for (int j = 0; j < KS; ++j) sel_b[j] = (j % 2) ? sel_a[j] : sel_a[j] + 5;  // odd entries kept, even ones new
    void *dsrc, *dstaged;
    int32_t *dsel, *dslot_tok, *dslot_of, *dftok, *dfslot, *dfcount;
    HIP_OK(hipMalloc(&dsrc, hsrc.size() * 2));
    HIP_OK(hipMalloc(&dstaged, (size_t)KS * row_bytes));
    HIP_OK(hipMalloc((void**)&dsel, KS * 4));
    HIP_OK(hipMalloc((void**)&dslot_tok, KS * 4));
    HIP_OK(hipMalloc((void**)&dslot_of, N * 4));
    HIP_OK(hipMalloc((void**)&dftok, KS * 4));
    HIP_OK(hipMalloc((void**)&dfslot, KS * 4));
    HIP_OK(hipMalloc((void**)&dfcount, 4));
    HIP_OK(hipMemcpy(dsrc, hsrc.data(), hsrc.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dslot_tok, minus.data(), KS * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dslot_of, minus_n.data(), N * 4, hipMemcpyHostToDevice));
    int32_t fetched[2] = {0, 0};
    for (int round = 0; round < 2; ++round) {
      HIP_OK(hipMemcpy(dsel, (round ? sel_b : sel_a).data(), KS * 4, hipMemcpyHostToDevice));
      OKV(okv_offload_plan(dsel, KS, dslot_tok, dslot_of, N, dftok, dfslot, dfcount, stream));
      OKV(okv_offload_fetch(dsrc, row_bytes, dftok, dfslot, dfcount, KS, dstaged, stream));
      HIP_OK(hipStreamSynchronize(stream));
      HIP_OK(hipMemcpy(&fetched[round], dfcount, 4, hipMemcpyDeviceToHost));
    }
    if (fetched[0] != KS || fetched[1] != KS / 2) {
      std::fprintf(stderr, "incremental staging fetched %d then %d rows, expected %d then %d\n", fetched[0], fetched[1], KS,
                   KS / 2);
      return 12;
    }
    std::vector<int32_t> slot_tok(KS);
    std::vector<uint16_t> staged((size_t)KS * row_bytes / 2);
    HIP_OK(hipMemcpy(slot_tok.data(), dslot_tok, KS * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(staged.data(), dstaged, staged.size() * 2, hipMemcpyDeviceToHost));
    std::vector<int32_t> held(slot_tok);
    std::sort(held.begin(), held.end());
    std::vector<int32_t> want_b(sel_b);
    std::sort(want_b.begin(), want_b.end());
    if (held != want_b) {
      std::fprintf(stderr, "the staged set is not the second selection\n");
      return 13;
    }
    for (int sl = 0; sl < KS; ++sl)
      if (std::memcmp(&staged[(size_t)sl * row_bytes / 2], &hsrc[(size_t)slot_tok[sl] * row_bytes / 2], row_bytes) != 0) {
        std::fprintf(stderr, "slot %d does not hold the row of token %d\n", sl, slot_tok[sl]);
        return 14;
      }
    for (void* p : {dsrc, dstaged, (void*)dsel, (void*)dslot_tok, (void*)dslot_of, (void*)dftok, (void*)dfslot, (void*)dfcount})
      HIP_OK(hipFree(p));
  }

  HIP_OK(hipStreamDestroy(stream));
  for (void* p : {dk, dv, dq, dout, dws, dgather, (void*)dscores, (void*)didx}) HIP_OK(hipFree(p));
  std::printf("abi smoke ok: %d rows, %d selected, score error %.2g\n", N, K_SEL, worst);
  return 0;
}
