// Composite entry points: tile plan, workspace carving, and the whole layer as
// one sequence of launches on the caller's stream.
#include "fr_common.h"
#include <cmath>

namespace fr {
namespace {

constexpr int64_t kAlign = 256;
int64_t aligned(int64_t bytes) { return round_up(bytes, kAlign); }

struct Carve {
  float* topk_w;
  int32_t* topk_ids;
  int32_t* sorted;
  int32_t* expert_ids;
  int32_t* npost;
  void* align_ws;
  int64_t align_ws_bytes;
  void* act;
  float* partial;
  float* tail;       // scratch for splitting the last round of 256-row tiles, or nullptr
  void* xq;          // fp8 layer only
  float* x_scale;
  void* actq;
  float* act_scale;
  int64_t total;
};

// the activated intermediate is stored in half precision also on the fp8 path
int act_elem_size(int) { return 2; }

Carve carve(void* base, int64_t M, int64_t H, int64_t F, int E, int topk, int dtype, const fr_moe_plan& p) {
  Carve c;
  const int64_t n = M * topk;
  char* b = static_cast<char*>(base);
  int64_t off = 0;
  auto take = [&](int64_t bytes) { char* r = b ? b + off : nullptr; off += aligned(bytes); return r; };
  c.topk_w = reinterpret_cast<float*>(take(n * 4));
  c.topk_ids = reinterpret_cast<int32_t*>(take(n * 4));
  c.sorted = reinterpret_cast<int32_t*>(take(p.sorted_len * 4));
  c.expert_ids = reinterpret_cast<int32_t*>(take((n + E) * 4));
  c.npost = reinterpret_cast<int32_t*>(take(4));
  c.align_ws_bytes = fr_moe_align_workspace_bytes(n, E);
  c.align_ws = take(c.align_ws_bytes);
  c.act = take(p.sorted_len * F * act_elem_size(dtype));
  c.partial = reinterpret_cast<float*>(take(static_cast<int64_t>(p.split_k) * n * H * 4));
  c.tail = p.tail_bytes > 0 ? reinterpret_cast<float*>(take(p.tail_bytes)) : nullptr;
  c.xq = nullptr; c.x_scale = nullptr; c.actq = nullptr; c.act_scale = nullptr;
  if (dtype == FR_FP8_E4M3) {
    c.xq = take(M * H);
    c.x_scale = reinterpret_cast<float*>(take(M * 4));
    c.actq = take(p.sorted_len * F);
    c.act_scale = reinterpret_cast<float*>(take(p.sorted_len * 4));
  }
  c.total = off;
  return c;
}

fr_moe_tunables g_tunables = {0, 0, 0, 0, 0};

int check_layer_shapes(const char* who, int64_t M, int64_t H, int64_t F, int E, int topk, int dtype) {
  FR_REQUIRE(dtype == FR_F16 || dtype == FR_BF16 || dtype == FR_FP8_E4M3, FR_E_DTYPE, "%s: dtype %d not in {f16, bf16, fp8_e4m3}", who, dtype);
  FR_REQUIRE(M >= 0 && H > 0 && F > 0, FR_E_SHAPE, "%s: M=%lld H=%lld F=%lld", who, (long long)M, (long long)H, (long long)F);
  FR_REQUIRE(E >= 1 && E <= 1024 && topk >= 1 && topk <= E, FR_E_SHAPE, "%s: E=%d topk=%d", who, E, topk);
  const int mult = dtype == FR_FP8_E4M3 ? 256 : 128;
  FR_REQUIRE(H % mult == 0 && F % mult == 0, FR_E_SHAPE, "%s: H=%lld and F=%lld must be multiples of %d", who, (long long)H, (long long)F, mult);
  FR_REQUIRE(M * topk < (int64_t(1) << 30), FR_E_SHAPE, "%s: M*topk too large", who);
  return FR_OK;
}

}  // namespace
const fr_moe_tunables& tunables() { return g_tunables; }
}  // namespace fr

using namespace fr;

extern "C" int fr_moe_set_tunables(const fr_moe_tunables* t) {
  if (!t) {
    g_tunables = fr_moe_tunables{0, 0, 0, 0, 0, 0};
    return FR_OK;
  }
  FR_REQUIRE(t->block == 0 || t->block == 16 || t->block == 32 || t->block == 64 || t->block == 128 || t->block == 160 || t->block == 256,
             FR_E_SHAPE, "fr_moe_set_tunables: block=%d not in {0, 16, 32, 64, 128, 160, 256}", t->block);
  FR_REQUIRE(t->split_k >= 0 && t->split_k <= 64, FR_E_SHAPE, "fr_moe_set_tunables: split_k=%d outside [0, 64]", t->split_k);
  FR_REQUIRE(t->group_m >= 0 && t->group_m <= 64, FR_E_SHAPE, "fr_moe_set_tunables: group_m=%d outside [0, 64]", t->group_m);
  FR_REQUIRE(t->no_tail_split == 0 || t->no_tail_split == 1, FR_E_SHAPE, "fr_moe_set_tunables: no_tail_split=%d", t->no_tail_split);
  FR_REQUIRE(t->epilogue_combine == 0 || t->epilogue_combine == 1, FR_E_SHAPE, "fr_moe_set_tunables: epilogue_combine=%d", t->epilogue_combine);
  FR_REQUIRE(t->no_quad == 0 || t->no_quad == 1, FR_E_SHAPE, "fr_moe_set_tunables: no_quad=%d", t->no_quad);
  g_tunables = *t;
  return FR_OK;
}

extern "C" int fr_moe_get_tunables(fr_moe_tunables* t) {
  FR_REQUIRE(t, FR_E_NULL, "fr_moe_get_tunables: null pointer");
  *t = g_tunables;
  return FR_OK;
}

extern "C" int fr_moe_get_plan(int64_t M, int64_t H, int64_t F, int E, int topk, int dtype, fr_moe_plan* plan) {
  FR_REQUIRE(plan, FR_E_NULL, "fr_moe_get_plan: null plan");
  dtype &= ~FR_W_TILED;  // the plan does not depend on the weight layout
  int rc = check_layer_shapes("fr_moe_get_plan", M, H, F, E, topk, dtype);
  if (rc != FR_OK) return rc;
  const int64_t n = M * topk;
  const double avg = static_cast<double>(n) / E;  // expected pairs per expert under uniform load
  // Routing block = token rows per GEMM tile.  Decode sizes want one block per expert
  // (weights are streamed once); from ~32 pairs per expert on, the 128-row MFMA tile
  // wins even with its padding, and 256 rows once runs are long enough to amortise it.
  // The 256-row tile's advantage grows with the K of the gate/up GEMM (its start-up per
  // tile is amortised over more K tiles); measured crossovers: 512..640 pairs per expert
  // at H = 4096 (F = 14336, E = 8: 2048 tokens 1380 us with 128 rows against 1435 with 256, 2560 tokens
  // 1810 against 1662).  At H = 2048 (F = 1408, E = 64, top-6: 32 and 22 K tiles per output tile) the 128-row
  // tile stays ahead as far as measured: 768 / 1536 pairs per expert 960 / 1738 us against 1002 / 1776.
  const double t256 = H >= 4096 ? 560.0 : (H <= 2048 ? 4096.0 : 4096.0 - (H - 2048) * (3536.0 / 2048.0));
  // Between 26 and 52 pairs per expert with a long gate/up K the 64-row tile wins: one block per expert
  // where 32-row blocks stream every expert's weights through the CUs twice, and half the MFMA and LDS work
  // of the 128-row tile (measured at H = 4096, F = 14336, E = 8: M = 112..192 4-6 % faster than either;
  // at H = 2048, F = 1408, E = 64 with skewed load it is slower than the 128-row tile, hence the K condition).
  int block;
  if (avg <= 8) block = 16;
  else if (avg < 26 || (avg < 32 && H < 4096)) block = 32;
  else if (avg < 52 && H >= 4096) block = 64;
  else if (avg < t256) block = 128;
  else block = 256;
  // 160-row blocks (a gate/up K of at least 32 K tiles): the same three-slot ring as the 128-row
  // tile with a quarter more rows per pass of an expert's weights through LDS.  Under uniform routing an expert
  // gets avg +- sqrt(avg) pairs, so with avg = 128, 256, 384, 512 every other expert needs one 128-row block more
  // than avg / 128; 160 rows absorb the spread.  Taken where the expected number of blocks per expert drops by an
  // eighth or more (1 / 1.15), or the expected rows the MFMAs multiply (whole half-blocks: a wavefront row is skipped when
  // all its rows are padding) by 2 %; measured on 8 experts, H = 4096, 128 / 160 / 256 rows:
  //   tokens  512  681 / 618         us      1536  1143 / 1112 / 1132       3072        1906 / 1939
  //           640  753 / 749                 1792  1236 / 1179 / 1192       4096        2433 / 2485
  //           768  715 / 743 (128 stays)     2048  1393 / 1386 / 1441       5120        2988 / 2975
  //           896  828 / 770                 2560  1706 / 1623 / 1685       6144        3507 / 3478
  //          1024  874 / 801                                                8192        4658 / 4512
  // With a 160-row candidate the 256-row tile takes over at 1200 pairs per expert (H >= 4096).  Below 112 pairs per expert one
  // block holds an expert either way and the smaller tile is cheaper (256 / 384 tokens: 548 / 556, 580 / 602 us);
  // with H = 1024 (16 K tiles) the 160-row tile loses (700 tokens: 85 / 96 us).
  // fp8 (16x16x128 MFMAs for this tile; its gate/up kernel spills 46 registers): only where a sixth of the blocks
  // go - 128 / 160 / 256 rows: 512 tokens 435 / 392, 1024: 543 / 505, 2560: 1145 / 1006 / 1063 us, but 2048: 853 / 877
  // / 899 - and below 900 pairs per expert (4096 tokens: 1506 against 1495 us with 256 rows).
  const bool two_byte = dtype == FR_BF16 || dtype == FR_F16;
  const double sigma = sqrt(avg * (1.0 - 1.0 / E)) + 1e-9;  // spread of an expert's pairs under uniform routing
  auto tail = [&](double x) { return 0.5 * erfc((x - avg) / (sigma * 1.4142135623730951)); };  // P(pairs of an expert > x)
  auto expected = [&](int rows) {  // expected multiples of `rows` that hold an expert's pairs
    double sum = 1.0;
    for (int k = 1; k * rows < avg + 8 * sigma; ++k) sum += tail(static_cast<double>(k) * rows);
    return sum;
  };
  if ((block == 128 || block == 256) && H >= 2048 && F >= 1024 && E <= 1022 && avg >= 112 &&
      avg < (H >= 4096 ? (two_byte ? 1200.0 : 900.0) : t256)) {
    const double b128 = expected(128), b160 = expected(160);
    const double c128 = expected(64) * 64, c160 = expected(80) * 80;
    const bool take160 = two_byte ? (b160 * 1.15 < b128 || c160 <= 0.98 * c128) : b160 * 1.2 < b128;
    if (take160) block = 160;
  }
  // 256 rows on the one-wavefront-per-SIMD kernel (2-byte operands, 16 K tiles or more in both GEMMs): a row of its
  // tiles costs about 8 % less than one of the 128- or 160-row tiles (4096 tokens 2365 against 2510 us with 160 rows,
  // 16384: 8494 / 9349), which pays wherever its coarser blocks do not add more rows than that.  Its rows: the mean
  // of whole blocks (the time of a tile) and whole half blocks (the wavefronts of an all-padding half idle: energy,
  // and the clock follows the energy).  Measured 160 / 256 rows on 8 experts, H = 4096: 1280 tokens 982 / 1040 us
  // (160 stays), 1536: 1148 / 1081, 1792: 1216 / 1102, 2048: 1395 / 1373, 2304: 1490 / 1626 (160 stays), 2560:
  // 1664 / 1647, 3072: 1973 / 1815, 5120: 3059 / 2911, 8192: 4804 / 4339.  Below 350 pairs per expert the smaller
  // tiles stream the weights faster (1024 tokens: 811 / 977 us).
  // With a short K (H = 2048, F = 1408, 64 experts: 32 and 22 K tiles per output tile) a tile's epilogue and hand-over
  // weigh more and the gain is smaller and later: 160 / 256 rows 4096 tokens (384 pairs per expert) 568 / 587 us,
  // 8192: 941 / 918, 16384: 1698 / 1637; taken from 700 pairs per expert on.
  // fp8 (32x32x64 MFMAs in that kernel; 16 K tiles are 2048 elements): 128 / 160 / 256 rows 2048 tokens 870 / - / 797 us,
  // 2560: - / 1040 / 941, 4096: - / 1554 / 1383 (1511 on the eight-wavefront kernel), 16384: 5386 -> 4882.
  if (!g_tunables.no_quad && (block == 128 || block == 160) && H >= 2048 && F >= 2048 / (two_byte ? 2 : 1) && E <= 1022 &&
      avg >= (H >= 4096 ? (two_byte ? 350.0 : 300.0) : 700.0)) {
    const double other = expected(block) * block;
    const double quad = 0.5 * (expected(256) * 256 + expected(128) * 128);
    // fp8 gains more per row (1280 tokens: 605 / 612 / 583 us with 128 / 160 / 256 rows, 2304: - / 882 / 870)
    if (quad <= (two_byte ? 1.08 : 1.18) * other) block = 256;
  }
  if (g_tunables.block) block = g_tunables.block;
  // the fp8 160-row tile exists in the persistent form only (five K tiles per K slice at least, 1022 experts at most)
  if (block == 160 && !two_byte && (H < 640 || F < 1024 || E > 1022)) block = 128;
  // Down projection: N = H gives few feature tiles, so K is split.
  const int bf = block == 16 ? 64 : (block == 32 ? 128 : 256);
  // expected token blocks: one per pair or per expert in the decode regime, else the expected blocks per expert
  const int64_t blocks = n <= E ? n : (block >= 128 ? static_cast<int64_t>(E * expected(block) + 0.5) : E);
  const int64_t tiles = blocks * ceil_div(H, bf);
  const int bk_elems = dtype == FR_FP8_E4M3 ? (block <= 32 ? 256 : 128) : (block == 16 ? 128 : 64);
  // 256-row tiles of 2-byte operands with a long K balance their last round themselves (its
  // tiles are cut along K over the idle workgroups); both GEMMs share the scratch for that.
  const int64_t tail_up = tail_scratch_bytes(block, dtype, H, F, true), tail_down = tail_scratch_bytes(block, dtype, F, H, false);
  int split = 1;
  if (tail_down > 0 && (tiles >= 192 || tiles <= 64)) {
    // whole rounds plus a split last round, or so few tiles that every one is cut into 4..8 slices;
    // in between (most of one round: no idle workgroups to cut for) all tiles are split alike
  } else if (block >= 128) {
    // one workgroup per CU: the split that minimises GEMM time (at ~0.9 PFLOP/s, stretched by how long the
    // busiest workgroup works: the persistent launch gives each of `sp` slices 256 / sp workgroups, rounded down
    // to whole XCD shares, and a workgroup does ceil(tiles / those) units of 1 / sp of a tile) plus the partial
    // traffic it causes (one 2-byte slice, or `split` fp32 slices, written and read back at ~4 TB/s: with many
    // pairs per weight byte that traffic decides).  Measured on 8 experts with one block each (128 tiles), down
    // projection with 1 / 2 / 3 / 4 slices: 384 tokens 185 / 174 / 212 / 196 us, 512 tokens 202 / 194 / 233 / 214.
    double best = 1e30;
    const double rows = static_cast<double>(blocks) * block, pairs = static_cast<double>(n);
    for (int sp = 1; sp <= 4; ++sp) {
      if (F / sp < 8 * bk_elems) break;
      const int64_t wgs = 256 / sp / 8 * 8;
      const double busiest = static_cast<double>(ceil_div(tiles, wgs)) / sp;  // in tiles
      const double fill = (static_cast<double>(tiles) / 256.0) / busiest;
      const double t_gemm = 2.0 * rows * H * F / 0.9e15 / (fill < 1.0 ? fill : 1.0);
      const double t_part = pairs * H * (sp == 1 ? 2.0 : 4.0 * sp) * 2.0 / 4e12;
      if (t_gemm + t_part < best) { best = t_gemm + t_part; split = sp; }
    }
  } else {
    // several workgroups per CU: aim at ~512 workgroups
    // (the 64-row tile runs one workgroup per CU: ~256)
    const int64_t target = block == 64 ? 256 : 512;
    while (split < 16 && tiles * split * 2 <= target && F / (split * 2) >= 8 * bk_elems) split *= 2;
    // between half a pair and one pair per expert: collisions are common (some experts get two rows,
    // some none) and the grid is partly filled by tiles of unequal luck; four slices even that out
    // (measured at 3 and 4 tokens on 8 experts, top-2: -9 % and -13 % on the down projection; with
    // fewer pairs the blocks are as many as the pairs and the rule above already fills the grid)
    if (n <= E && 2 * n > E && tiles <= 512)
      while (split < 4 && F / (split * 2) >= 8 * bk_elems) split *= 2;
  }
  int64_t tail_bytes = tail_up > tail_down ? tail_up : tail_down;
  if (g_tunables.split_k) {  // as many slices as asked for, as far as every slice keeps 8 K tiles
    split = g_tunables.split_k;
    while (split > 1 && F / split < 8 * bk_elems) --split;
  }
  if (g_tunables.no_tail_split) tail_bytes = 0;
  plan->block = block;
  plan->split_k = split;
  plan->sorted_len = n + static_cast<int64_t>(E) * (block - 1);
  plan->tail_bytes = tail_bytes;
  plan->workspace_bytes = carve(nullptr, M, H, F, E, topk, dtype, *plan).total;
  return FR_OK;
}

namespace fr {
namespace {
// top-k gating of the logits and the routing arrays of the result: one launch for small
// batches, gating then align otherwise.  qx (fp8 layer): the bf16 token rows [M, H], quantised per row into
// c.xq / c.x_scale - by the same launch for small batches, by one of its own otherwise.
int route_and_align(const void* logits, int logits_dtype, int64_t M, int E, int topk, int renormalize, int block,
                    const Carve& c, const void* qx, int64_t H, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (route_align_fits(M, E, topk))
    return route_align_small(logits, logits_dtype, M, E, topk, renormalize, block, c.topk_w, c.topk_ids, c.sorted,
                             c.expert_ids, c.npost, qx, H, c.xq, c.x_scale, st);
  int rc = fr_gating_topk(logits, logits_dtype, M, E, E, topk, renormalize, c.topk_w, c.topk_ids, stream);
  if (rc != FR_OK) return rc;
  rc = fr_moe_align(c.topk_ids, FR_I32, M * topk, E, block, c.sorted, c.expert_ids, c.npost, c.align_ws, c.align_ws_bytes, stream);
  if (rc != FR_OK || !qx) return rc;
  return quant_rows(qx, FR_BF16, M, nullptr, H, H, c.xq, c.x_scale, st);
}
}  // namespace
}  // namespace fr

extern "C" int fr_fused_experts(const void* x, const void* w1, const void* w2, const float* topk_weights,
                                const int32_t* topk_ids, int64_t M, int64_t H, int64_t F, int E, int topk,
                                int dtype, void* out, void* workspace, int64_t workspace_bytes, void* stream) {
  fr_moe_plan p;
  int rc = fr_moe_get_plan(M, H, F, E, topk, dtype, &p);
  if (rc != FR_OK) return rc;
  if (M == 0) return FR_OK;
  FR_REQUIRE(x && w1 && w2 && topk_weights && topk_ids && out, FR_E_NULL, "fr_fused_experts: null pointer");
  FR_REQUIRE(workspace && workspace_bytes >= p.workspace_bytes, FR_E_WORKSPACE, "fr_fused_experts: workspace %lld < %lld bytes", (long long)workspace_bytes, (long long)p.workspace_bytes);
  FR_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, FR_E_ALIGN, "fr_fused_experts: workspace must be 256-byte aligned");
  Carve c = carve(workspace, M, H, F, E, topk, dtype & ~FR_W_TILED, p);
  rc = fr_moe_align(topk_ids, FR_I32, M * topk, E, p.block, c.sorted, c.expert_ids, c.npost, c.align_ws, c.align_ws_bytes, stream);
  if (rc != FR_OK) return rc;
  rc = fr_moe_gateup_silu(x, w1, c.sorted, c.expert_ids, c.npost, M, H, F, E, topk, p.block, dtype, c.act, c.tail, stream);
  if (rc != FR_OK) return rc;
  return down_impl(c.act, nullptr, w2, nullptr, topk_weights, c.sorted, c.expert_ids, c.npost, M, H, F, E, topk, p.block,
                   p.split_k, dtype & ~FR_W_TILED, dtype & ~FR_W_TILED, c.partial, out, c.tail, static_cast<hipStream_t>(stream),
                   "fr_fused_experts", (dtype & FR_W2_TILED) ? 1 : 0, topk_ids);
}

extern "C" int fr_fused_moe(const void* x, const void* w1, const void* w2, const void* logits, int logits_dtype,
                            int64_t M, int64_t H, int64_t F, int E, int topk, int renormalize, int dtype,
                            void* out, void* workspace, int64_t workspace_bytes, void* stream) {
  fr_moe_plan p;
  int rc = fr_moe_get_plan(M, H, F, E, topk, dtype, &p);
  if (rc != FR_OK) return rc;
  if (M == 0) return FR_OK;
  FR_REQUIRE(x && w1 && w2 && logits && out, FR_E_NULL, "fr_fused_moe: null pointer");
  FR_REQUIRE(workspace && workspace_bytes >= p.workspace_bytes, FR_E_WORKSPACE, "fr_fused_moe: workspace %lld < %lld bytes", (long long)workspace_bytes, (long long)p.workspace_bytes);
  FR_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, FR_E_ALIGN, "fr_fused_moe: workspace must be 256-byte aligned");
  Carve c = carve(workspace, M, H, F, E, topk, dtype & ~FR_W_TILED, p);
  // a handful of tokens: the gate/up launch gates and sorts by itself (row-major weights only)
  rc = (dtype & FR_W1_TILED) ? 1
                            : gateup_rows_routed(x, w1, logits, logits_dtype, M, H, F, E, topk, renormalize, p.block, dtype, c.act, c.topk_w,
                                                 c.topk_ids, c.sorted, c.expert_ids, c.npost, static_cast<hipStream_t>(stream));
  if (rc < 0) return rc;
  if (rc == 1) {
    rc = route_and_align(logits, logits_dtype, M, E, topk, renormalize, p.block, c, nullptr, H, stream);
    if (rc != FR_OK) return rc;
    rc = fr_moe_gateup_silu(x, w1, c.sorted, c.expert_ids, c.npost, M, H, F, E, topk, p.block, dtype, c.act, c.tail, stream);
    if (rc != FR_OK) return rc;
  }
  return down_impl(c.act, nullptr, w2, nullptr, c.topk_w, c.sorted, c.expert_ids, c.npost, M, H, F, E, topk, p.block,
                   p.split_k, dtype & ~FR_W_TILED, dtype & ~FR_W_TILED, c.partial, out, c.tail, static_cast<hipStream_t>(stream),
                   "fr_fused_moe", (dtype & FR_W2_TILED) ? 1 : 0, c.topk_ids);
}

extern "C" int fr_fused_moe_fp8(const void* x, int x_dtype, const void* w1q, const float* w1_scale, const void* w2q,
                                const float* w2_scale, const void* logits, int logits_dtype, int64_t M, int64_t H,
                                int64_t F, int E, int topk, int renormalize, void* out, void* workspace,
                                int64_t workspace_bytes, void* stream) {
  fr_moe_plan p;
  int rc = fr_moe_get_plan(M, H, F, E, topk, FR_FP8_E4M3, &p);
  if (rc != FR_OK) return rc;
  if (M == 0) return FR_OK;
  const int w2_flag = x_dtype & FR_W2_TILED;
  x_dtype &= ~FR_W_TILED;
  FR_REQUIRE(x_dtype == FR_BF16, FR_E_DTYPE, "fr_fused_moe_fp8: activations must be bf16 (dtype %d)", x_dtype);
  FR_REQUIRE(x && w1q && w1_scale && w2q && w2_scale && logits && out, FR_E_NULL, "fr_fused_moe_fp8: null pointer");
  FR_REQUIRE(workspace && workspace_bytes >= p.workspace_bytes, FR_E_WORKSPACE, "fr_fused_moe_fp8: workspace %lld < %lld bytes", (long long)workspace_bytes, (long long)p.workspace_bytes);
  FR_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, FR_E_ALIGN, "fr_fused_moe_fp8: workspace must be 256-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  Carve c = carve(workspace, M, H, F, E, topk, FR_FP8_E4M3, p);
  rc = route_and_align(logits, logits_dtype, M, E, topk, renormalize, p.block, c, x, H, stream);
  if (rc != FR_OK) return rc;
  rc = fr_moe_gateup_silu_fp8(c.xq, c.x_scale, w1q, w1_scale, c.sorted, c.expert_ids, c.npost, M, H, F, E, topk, p.block, c.act, stream);
  if (rc != FR_OK) return rc;
  rc = quant_rows(c.act, FR_BF16, p.sorted_len, c.npost, F, F, c.actq, c.act_scale, st);
  if (rc != FR_OK) return rc;
  return fr_moe_down_combine_fp8(c.actq, c.act_scale, w2q, w2_scale, c.topk_w, c.sorted, c.expert_ids, c.npost, M, H, F, E,
                                 topk, p.block, p.split_k, x_dtype | w2_flag, c.partial, out, c.tail, stream);
}

// ---- one entry point that allocates nothing ------------------------------------
// The layer's scratch lives in a device array of this library instead of a caller's buffer.
// Host code may not pass the array's name to a kernel (on the host it is a stand-in, not a
// device address): its address on the current device is looked up once per device and kept.
namespace fr {
namespace {
constexpr int64_t kStaticScratchBytes = int64_t(64) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

int static_scratch(void** out) {
  constexpr int kMaxDevices = 64;
  static void* ptrs[kMaxDevices] = {};  // per device; two threads racing here store the same address
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(FR_E_NO_DEVICE, "fr_fused_moe_noalloc: device %d (%s)", dev, hipGetErrorString(e));
  if (!ptrs[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      return fail(FR_E_NO_DEVICE, "fr_fused_moe_noalloc: hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    }
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return FR_OK;
}
}  // namespace
int prepare_static_scratch() {
  void* p = nullptr;
  return static_scratch(&p);
}
}  // namespace fr

extern "C" int fr_fused_moe_noalloc(const void* x, const void* w1, const void* w2, const void* logits, int logits_dtype,
                                    int64_t M, int64_t H, int64_t F, int E, int topk, int renormalize, int dtype,
                                    void* out, void* stream) {
  fr_moe_plan p;
  int rc = fr_moe_get_plan(M, H, F, E, topk, dtype, &p);
  if (rc != FR_OK) return rc;
  FR_REQUIRE((dtype & ~FR_W_TILED) == FR_F16 || (dtype & ~FR_W_TILED) == FR_BF16, FR_E_DTYPE, "fr_fused_moe_noalloc: dtype %d not in {f16, bf16}", dtype);
  FR_REQUIRE(p.workspace_bytes <= kStaticScratchBytes, FR_E_WORKSPACE,
             "fr_fused_moe_noalloc: these sizes need %lld bytes of scratch, the library's static scratch holds %lld; use fr_fused_moe with a workspace",
             (long long)p.workspace_bytes, (long long)kStaticScratchBytes);
  if (M == 0) return FR_OK;
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc != FR_OK) return rc;
  return fr_fused_moe(x, w1, w2, logits, logits_dtype, M, H, F, E, topk, renormalize, dtype, out, ws, kStaticScratchBytes, stream);
}
