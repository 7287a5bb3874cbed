// Status strings, argument validation and workspace sizing of libomnikv_hip.so.
#include <stdarg.h>
#include <string.h>

#include <algorithm>

#include "okv_internal.h"

namespace okv {

static thread_local char g_last_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Rows per split: enough blocks to fill 256 CUs several times over for long
// contexts, never below one 64-row tile group.
std::atomic<int> g_split_rows_override{0};

static int num_compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;  // MI355X
  }
  return cus;
}

// Local data share a workgroup may ask for on this device.
int lds_bytes_per_workgroup() {
  static int bytes = 0;
  if (bytes == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && n > 0)
      bytes = n;
    else
      bytes = 64 * 1024;
  }
  return bytes;
}

// Rows per split.  The pass is bandwidth-bound, so the grid is sized to what the chip holds at
// once, every workgroup getting the same share of rows: all of them start together and finish
// together, in one round when the split fits the row cap, else in the fewest equal rounds.
// The attention kernels hold two workgroups per CU (their registers allow two waves per SIMD);
// scoring alone could hold five and does best sized for three (measured at 128K: 50.6 us against
// 53.1 sized for six).  A scored split stages its logits in LDS and hands them over in one burst
// at its end, and every round of workgroups ends in such a burst, so the cap on its rows is what
// the LDS of a CU lets the resident workgroups stage: 160 KB shared by two attention workgroups,
// each with 16 KB of K staging and its logits (one row per q head of the group, or one per kv head
// when the pass folds the group itself -- kind 3).
static int choose_split_rows(int batch, int hq, int hkv, int total_rows, bool with_v,
                             bool with_logits, int kind) {
  const int forced = g_split_rows_override.load(std::memory_order_relaxed);
  if (forced > 0) return forced;
  // a batch is sized by its longest request, so ragged ones fill less than the grid suggests:
  // three and six per CU there (measured on 16 requests of 8K..32K tokens)
  // kind 2: the dense pass that carries a query window needs more than half a SIMD's registers per wave, so
  // one workgroup per CU is resident
  const int group = kind == 3 ? 1 : hkv > 0 && hq >= hkv ? hq / hkv : 1;
  const int64_t work = (int64_t)(total_rows > 0 ? total_rows : 1) * hkv * (batch > 0 ? batch : 1);
  // rows per split and rounds of workgroups for `per_cu` resident workgroups whose splits stage at
  // most `logit_bytes` of logits
  auto plan = [&](int per_cu, int64_t logit_bytes, int64_t* rounds_out) -> int {
    const int64_t capacity = (int64_t)num_compute_units() * per_cu;
    const int64_t cap_rows = with_logits ? std::min<int64_t>(logit_bytes / (4 * group) / 64 * 64, 8192) : kind == 2 ? 8192 : 4096;
    // a sparse layer's share is a few 16-row tiles per wave: cut to the tile, so that all CUs hold two
    // workgroups (137 -> 144 rows at 8781 selected rows, where rounding to 64 left 112 CUs with two
    // workgroups of 192 and 144 CUs with one)
    const int64_t gran = kind == 1 && batch <= 1 ? 16 : 64;
    for (int64_t rounds = 1;; ++rounds) {
      int64_t rows = (work + rounds * capacity - 1) / (rounds * capacity);
      rows = (rows + gran - 1) / gran * gran;
      if (rows < 64) rows = 64;
      if (rounds == 1 && with_v && batch > 1 && rows <= 128) {
        // a short pass is a chain of latencies: fewer, fatter workgroups
        rows = (work + capacity * 2 / 3 - 1) / (capacity * 2 / 3);
        rows = (rows + 63) / 64 * 64;
      }
      if (rows <= cap_rows) {
        *rounds_out = rounds;
        return (int)rows;
      }
    }
  };
  const int64_t three_share = 33 * 1024;  // logits three resident workgroups leave each other (next to their K staging)
  const int64_t two_share = std::max<int64_t>(three_share, std::min<int64_t>(lds_bytes_per_workgroup(), 80 * 1024) - 17 * 1024);
  int64_t rounds = 0;
  if (kind == 2) return plan(1, three_share, &rounds);
  if (batch > 1) return plan(with_v ? 3 : 6, three_share, &rounds);
  if (with_v) return plan(2, two_share, &rounds);
  // scoring alone: sized for three per CU unless two, with their longer splits, save a round of bursts
  int64_t rounds2 = 0;
  const int rows3 = plan(3, three_share, &rounds), rows2 = plan(2, two_share, &rounds2);
  return with_logits && rounds2 < rounds ? rows2 : rows3;
}

size_t attn_workspace_bytes(int batch, int hq, int hkv, int d, int max_main, int max_tail,
                            int max_score, bool with_v, bool with_logits, int* split_rows,
                            int* max_splits, int kind) {
  int L = max_main + max_tail;
  int C = choose_split_rows(batch, hq, hkv, L, with_v, with_logits, kind);
  int S = (L + C - 1) / C + (max_score > 0 ? 1 : 0);
  if (S < 1) S = 1;
  if (split_rows) *split_rows = C;
  if (max_splits) *max_splits = S;
  size_t bytes = 0;
  if (with_v) bytes += align_up((size_t)batch * hq * S * d * sizeof(float), 256);
  bytes += align_up((size_t)batch * hq * S * sizeof(float), 256);
  if (with_logits) {
    size_t ls = align_up((size_t)max_score, 64);
    bytes += align_up((size_t)batch * hq * ls * sizeof(float), 256);
  }
  bytes += align_up((size_t)batch * hq * sizeof(float), 256);
  return bytes + 256;
}

int carve_attn_workspace(void* ws, size_t ws_bytes, int batch, int hq, int hkv, int d,
                         int max_main, int max_tail, int max_score, bool with_v,
                         bool with_logits, AttnWorkspace* out, int kind) {
  int C = 0, S = 0;
  size_t need = attn_workspace_bytes(batch, hq, hkv, d, max_main, max_tail, max_score, with_v,
                                     with_logits, &C, &S, kind);
  OKV_REQUIRE(ws != nullptr, OKV_ERR_INVALID, "workspace pointer is NULL");
  OKV_REQUIRE(ws_bytes >= need, OKV_ERR_WORKSPACE, "workspace too small: have %zu, need %zu",
              ws_bytes, need);
  char* p = (char*)align_up((size_t)ws, 256);
  memset(out, 0, sizeof(*out));
  out->split_rows = C;
  out->max_splits = S;
  out->logit_heads = hq;
  if (with_v) {
    out->part_o = (float*)p;
    p += align_up((size_t)batch * hq * S * d * sizeof(float), 256);
  }
  out->part_lse = (float*)p;
  p += align_up((size_t)batch * hq * S * sizeof(float), 256);
  if (with_logits) {
    out->logits_stride = (int64_t)align_up((size_t)max_score, 64);
    out->logits = (float*)p;
    p += align_up((size_t)batch * hq * out->logits_stride * sizeof(float), 256);
  }
  out->score_lse = (float*)p;
  return OKV_OK;
}

size_t window_workspace_bytes(int batch, int hkv, int max_len);
size_t dense_window_workspace_bytes(int batch, int hq, int hkv, int d, int max_seq_len, int max_score_len);

int validate_layout(const okv_kv_layout_t* layout, const void* k_base, const void* v_base) {
  OKV_REQUIRE(layout != nullptr, OKV_ERR_INVALID, "layout is NULL");
  OKV_REQUIRE(k_base != nullptr, OKV_ERR_INVALID, "k_base is NULL");
  OKV_REQUIRE(layout->dtype == OKV_F32 || layout->dtype == OKV_BF16 || layout->dtype == OKV_F16,
              OKV_ERR_UNSUPPORTED, "dtype %d not supported", layout->dtype);
  OKV_REQUIRE(layout->head_dim == 128, OKV_ERR_UNSUPPORTED,
              "head_dim %d not supported (kernels are built for 128)", layout->head_dim);
  OKV_REQUIRE(layout->num_kv_heads >= 1 && layout->num_q_heads >= layout->num_kv_heads &&
                  layout->num_q_heads % layout->num_kv_heads == 0,
              OKV_ERR_INVALID, "bad head counts q=%d kv=%d", layout->num_q_heads,
              layout->num_kv_heads);
  int group = layout->num_q_heads / layout->num_kv_heads;
  OKV_REQUIRE(group == 1 || group == 2 || group == 4 || group == 8, OKV_ERR_UNSUPPORTED,
              "GQA group size %d not supported (1, 2, 4, 8)", group);
  OKV_REQUIRE(layout->token_stride % 8 == 0 && layout->head_stride % 8 == 0 &&
                  layout->batch_stride % 8 == 0 && layout->page_stride % 8 == 0,
              OKV_ERR_INVALID, "strides must be multiples of 8 elements");
  OKV_REQUIRE(((uintptr_t)k_base & 15) == 0 && ((uintptr_t)v_base & 15) == 0, OKV_ERR_INVALID,
              "K/V base pointers must be 16-byte aligned");
  if (layout->page_table) {
    OKV_REQUIRE(layout->page_size >= 1, OKV_ERR_INVALID, "page_size must be >= 1");
    OKV_REQUIRE(layout->page_table_stride >= 1, OKV_ERR_INVALID, "page_table_stride must be >= 1");
  }
  return OKV_OK;
}

}  // namespace okv

extern "C" {

const char* okv_strerror(int status) {
  switch (status) {
    case OKV_OK: return "ok";
    case OKV_ERR_INVALID: return "invalid argument";
    case OKV_ERR_UNSUPPORTED: return "unsupported geometry or dtype";
    case OKV_ERR_WORKSPACE: return "workspace too small";
    case OKV_ERR_HIP: return "HIP runtime error";
    default: return "unknown status";
  }
}

const char* okv_last_error(void) { return okv::g_last_error; }

int okv_version(void) { return 1; }

int okv_workspace_bytes(int op, const okv_shape_t* s, size_t* out_bytes) {
  OKV_REQUIRE(s != nullptr && out_bytes != nullptr, OKV_ERR_INVALID, "NULL argument");
  OKV_REQUIRE(s->batch >= 1, OKV_ERR_INVALID, "batch must be >= 1");
  OKV_REQUIRE(op == OKV_OP_TOPK || (s->num_q_heads >= 1 && s->num_kv_heads >= 1 && s->head_dim >= 1),
              OKV_ERR_INVALID, "head counts and head_dim must be >= 1");
  switch (op) {
    case OKV_OP_SCORE:
      *out_bytes = okv::attn_workspace_bytes(s->batch, s->num_q_heads, s->num_kv_heads, s->head_dim,
                                             s->max_seq_len, 0, s->max_seq_len, false, true,
                                             nullptr, nullptr);
      return OKV_OK;
    case OKV_OP_DENSE_ATTN:
      *out_bytes = okv::attn_workspace_bytes(s->batch, s->num_q_heads, s->num_kv_heads, s->head_dim,
                                             s->max_seq_len, 0,
                                             s->with_scores ? s->max_seq_len : 0, true,
                                             s->with_scores != 0, nullptr, nullptr);
      return OKV_OK;
    case OKV_OP_SPARSE_ATTN:
      *out_bytes = okv::attn_workspace_bytes(s->batch, s->num_q_heads, s->num_kv_heads, s->head_dim,
                                             s->max_seq_len, s->max_tail_len, 0, true, false,
                                             nullptr, nullptr, true);
      return OKV_OK;
    case OKV_OP_TOPK:
      *out_bytes = okv::topk_mb_workspace_bytes(s->batch, s->max_seq_len);
      return OKV_OK;
    case OKV_OP_DENSE_ATTN_SELECT: {  // the attention's part as the call carves it, then the selection's
      const size_t attn = okv::attn_workspace_bytes(s->batch, s->num_q_heads, s->num_kv_heads, s->head_dim,
                                                    s->max_seq_len, 0, s->max_seq_len, true, true, nullptr,
                                                    nullptr);
      *out_bytes = ((attn + 255) & ~(size_t)255) + okv::topk_mb_workspace_bytes(s->batch, s->max_seq_len);
      return OKV_OK;
    }
    case OKV_OP_DENSE_ATTN_WINDOW:
      *out_bytes = okv::dense_window_workspace_bytes(s->batch, s->num_q_heads, s->num_kv_heads, s->head_dim,
                                                     s->max_seq_len, s->max_seq_len);
      return OKV_OK;
    case OKV_OP_SCORE_WINDOW:
      *out_bytes = okv::window_workspace_bytes(s->batch, s->num_kv_heads, s->max_seq_len);
      return OKV_OK;
    default:
      okv::set_error("unknown op %d", op);
      return OKV_ERR_INVALID;
  }
}

}  // extern "C"
