// Host-side sanitizer run of the format builders through the C-ABI (no GPU): random matrices through every skeleton,
// dense operators, the forms of the tile template, kernel source generation.
#include "alphasparse_amd.h"
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <set>
#include <vector>
struct Coo { uint64_t rows, cols; std::vector<uint64_t> r, c; std::vector<double> v; };
static Coo make(std::mt19937_64 &g, int law) {
  Coo m;
  m.rows = 200 + g() % 6000;
  std::vector<uint64_t> len(m.rows);
  for (auto &l : len) {
    if (law == 0) l = 1 + g() % 24;
    else if (law == 1) { double u = (g() % 1000000 + 1) / 1e6; l = std::min<uint64_t>(1 + (uint64_t)(1.0 / (u * u) * 0.5), std::min<uint64_t>(m.rows, 2500)); }
    else if (law == 2) l = (g() % 3) ? 1 + g() % 3 : 20 + g() % 300;
    else l = 27;
  }
  uint64_t mx = *std::max_element(len.begin(), len.end());
  m.cols = std::max<uint64_t>(mx, (g() % 2) ? m.rows : 3 * m.rows + 1);
  for (uint64_t i = 0; i < m.rows; i++) {
    std::set<uint64_t> cs;
    if (law == 3) { uint64_t base = (i / 3) * 3; for (int k = 0; k < 9; k++) { uint64_t b = (base + 3 * (g() % 40)) % (m.cols - 3); b = b / 3 * 3; for (int q = 0; q < 3; q++) cs.insert(b + q); } }
    else while (cs.size() < len[i]) cs.insert(g() % m.cols);
    for (uint64_t c : cs) { m.r.push_back(i); m.c.push_back(c); m.v.push_back((double)(g() % 2000) / 1000.0 - 1.0); }
  }
  return m;
}
struct Step { int strategy; long p[4]; };
static int fails = 0, built = 0;
#define CK(x) do { if ((x) < 0) { fails++; } } while (0)
int main(int argc, char **argv) {
  int n_cases = argc > 1 ? atoi(argv[1]) : 40;
  std::mt19937_64 g(12345);
  for (int cs = 0; cs < n_cases; cs++) {
    int law = cs % 4;
    Coo c = make(g, law);
    int vdt = (g() % 2) ? AS_DOUBLE : AS_FLOAT;
    for (int sk = 0; sk < 14; sk++) {
      as_matrix *m = as_matrix_from_coo(c.rows, c.cols, c.r.size(), c.r.data(), c.c.data(), c.v.data(), vdt, 64);
      if (!m) { printf("from_coo failed: %s\n", as_last_error()); return 1; }
      long none[4] = {0, 0, 0, 0};
      int dense = (int)(g() % 4);
      if (dense >= 1) { long p[4] = {1, 0, 0, 0}; CK(as_execute_strategy(m, AS_DENSE_ROW_COARSE_SORT_FIXED, -1, p)); }
      if (dense == 2) { long p[4] = {(long)(8 + g() % 40), 2048, 4, 0}; CK(as_execute_strategy(m, AS_DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, p)); }
      if (dense == 3) { long p[4] = {16, 16, 2, 0}; CK(as_execute_strategy(m, AS_DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, p)); }
      CK(as_execute_strategy(m, AS_COMPRESS_NONE, -1, none));
      uint64_t info[8];
      as_matrix_info(m, info);
      std::vector<Step> steps;
      std::vector<int> tpl;
      long a = 1 << (5 + g() % 3), s4 = 3 + g() % 8;
      switch (sk) {
        case 0: steps = {{AS_COMPRESSED_ROW_PADDING_DIRECT, {a, 1}}, {AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, {a}}, {AS_COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE, {}}}; tpl = {AS_DIRECT_ATOM_TEMPLATE_WARP_COMPRESS}; break;
        case 1: steps = {{AS_COMPRESSED_ROW_PADDING_DIRECT, {64, 1}}, {AS_COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE, {}}}; tpl = {AS_DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS}; break;
        case 2: steps = {{AS_COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT, {(long)(2 + g() % 6)}}}; tpl = {AS_UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE, AS_UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE}; break;
        case 3: steps = {{AS_COMPRESSED_WARP_LEVEL_COL_DIV_FIXED, {a}}}; tpl = {AS_DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE}; break;
        case 4: steps = {{AS_COMPRESSED_ROW_PADDING_DIRECT, {4, 1}}, {AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, {4}}, {AS_COMPRESSED_WARP_LEVEL_COL_DIV_FIXED, {32}}}; tpl = {AS_SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE}; break;
        case 5: steps = {{AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ, {512}}, {AS_COMPRESSED_WARP_LEVEL_COL_DIV_FIXED, {a}}}; tpl = {AS_SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE}; break;
        case 6: steps = {{AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED, {(long)(64 << (g() % 4))}}}; tpl = {AS_SHARED_MEMORY_LONG_ROW_TEMPLATE}; break;
        case 7: steps = {{AS_COMPRESSED_ROW_PADDING_DIRECT, {a, 1}}, {AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, {a}}, {AS_COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED, {s4}}}; tpl = {AS_SHARED_MEMORY_TEMPLATE_WARP_COMPRESS}; break;
        case 8: steps = {{AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ, {896}}, {AS_COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED, {s4}}}; tpl = {AS_SHARED_MEMORY_TEMPLATE_WARP_COMPRESS}; break;
        case 9: steps = {{AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, {a}}, {AS_COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY, {8}}, {AS_COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE, {}}}; tpl = {AS_DIRECT_ATOM_TEMPLATE}; break;
        case 10: steps = {{AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ, {512}}, {AS_COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY, {8}}, {AS_COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED, {s4}}}; tpl = {AS_SHARED_MEMORY_TEMPLATE}; break;
        case 11: steps = {{AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE, {(long)(128 << (g() % 6))}}}; tpl = {AS_SHARED_MEMORY_X_SLICE_TEMPLATE}; break;
        case 12: steps = {{AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE, {(long)(128 << (g() % 7)), (long)(24 << (g() % 8)), (long)(100 + g() % 8000)}}}; tpl = {AS_SHARED_MEMORY_TILE_TEMPLATE}; break;
        default: steps = {{AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE, {(long)(128 << (g() % 7)), (long)(64 << (g() % 7)), (long)(100 + g() % 8000)}}}; tpl = {AS_SHARED_MEMORY_PRODUCT_BIN_TEMPLATE}; break;
      }
      bool ok = true;
      for (uint64_t sub = 0; sub < info[4] && ok; sub++) {   
        for (auto &st : steps) if (as_execute_strategy(m, st.strategy, (int64_t)sub, st.p) < 0) { ok = false; break; }
        if (ok && as_complete_blocking(m, (int64_t)sub) < 0) ok = false;
      }
      if (ok) {
        for (int tp : tpl) {
          as_builder *b = as_builder_create(m);
          bool set = true;
          for (uint64_t sub = 0; sub < info[4]; sub++)
            if (as_template_is_supported(m, (int64_t)sub, tp) != 1 || as_builder_set_template(b, (int64_t)sub, tp) < 0) { set = false; break; }
          if (set) {
            if (tp == AS_SHARED_MEMORY_TILE_TEMPLATE) {
              if (g() % 2) as_builder_set_column_runs(b, 0);
              if (as_builder_set_row_ownership(b, 0) == 1 && law == 3 && dense == 0) as_builder_set_row_blocks(b, 0, 3);
            }
            for (uint64_t sub = 0; sub < info[4]; sub++) as_builder_compress(b, (int64_t)sub);
            if (g() % 2) as_builder_set_launch(b, 0, 0, 64 << (g() % 5), 0, 0);
            as_builder_set_serial_launch(b, 1);
            const char *src = as_builder_kernel_source(b);
            if (src) built++; else { fails++; printf("source failed (case %d skeleton %d): %s\n", cs, sk, as_last_error()); }
            as_builder_algorithmic_bytes(b);
          }
          as_builder_free(b);
        }
      }
      as_matrix_free(m);
    }
    {  // two strips: tile + product-bin, fused / carried sources; sub-block division; column division; empty rows removed
      as_matrix *m = as_matrix_from_coo(c.rows, c.cols, c.r.size(), c.r.data(), c.c.data(), c.v.data(), vdt, 64);
      long p1[4] = {1, 0, 0, 0}, p2[4] = {16, 16, 2, 0}, none[4] = {0, 0, 0, 0};
      as_execute_strategy(m, AS_DENSE_ROW_COARSE_SORT_FIXED, -1, p1);
      as_execute_strategy(m, AS_DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, p2);
      as_execute_strategy(m, AS_COMPRESS_NONE, -1, none);
      uint64_t info[8];
      as_matrix_info(m, info);
      if (info[4] == 2) {
        long t1[4] = {(long)(256 << (g() % 6)), (long)(64 << (g() % 6)), 2048, 0}, t2[4] = {(long)(256 << (g() % 6)), (long)(256 << (g() % 5)), 2048, 0};
        if (as_execute_strategy(m, AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE, 0, t1) == 0 && as_complete_blocking(m, 0) == 0 &&
            as_execute_strategy(m, AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE, 1, t2) == 0 && as_complete_blocking(m, 1) == 0 &&
            as_template_is_supported(m, 0, AS_SHARED_MEMORY_TILE_TEMPLATE) == 1 && as_template_is_supported(m, 1, AS_SHARED_MEMORY_PRODUCT_BIN_TEMPLATE) == 1) {
          as_builder *b = as_builder_create(m);
          as_builder_set_template(b, 0, AS_SHARED_MEMORY_TILE_TEMPLATE);
          as_builder_set_template(b, 1, AS_SHARED_MEMORY_PRODUCT_BIN_TEMPLATE);
          long th = 256 << (g() % 3);
          as_builder_set_launch(b, 0, 0, th, 0, 0);
          as_builder_set_launch(b, 1, 0, (g() % 2) ? th : 1024, 0, 0);
          as_builder_set_serial_launch(b, 1);
          if (as_builder_kernel_source(b)) built++; else { fails++; printf("two-strip source failed: %s\n", as_last_error()); }
          as_builder_set_fuse_launches(b, 0);
          if (as_builder_kernel_source(b)) built++; else fails++;
          as_builder_set_finish_carry(b, 0);
          if (as_builder_kernel_source(b)) built++; else fails++;
          as_builder_free(b);
        }
      }
      as_matrix_free(m);
      // division of a sub-block, column bands
      m = as_matrix_from_coo(c.rows, c.cols, c.r.size(), c.r.data(), c.c.data(), c.v.data(), vdt, 64);
      long d[4] = {(long)(c.rows / 3 + 1), 0, 0, 0};
      long sc2[2] = {0, (long)(c.rows / 7 + 1)};
      uint64_t pos[3] = {0, c.rows / 3, c.rows};
      as_execute_node(m, AS_DENSE_ROW_DIV, -1, nullptr, 0, pos, 3, nullptr, 0);
      as_execute_node(m, AS_DENSE_ROW_DIV, -1, sc2, 2, nullptr, 0, nullptr, 0);
      long cd[2] = {(long)(c.cols / 5 + 1), 1};
      as_execute_node(m, AS_DENSE_FIXED_COL_DIV, -1, cd, 2, nullptr, 0, nullptr, 0);
      as_execute_strategy(m, AS_COMPRESS_NONE, -1, none);
      as_matrix_info(m, info);
      for (uint64_t sub = 0; sub < info[4]; sub++) {
        long e[4] = {64, 1, 0, 0};
        as_execute_strategy(m, AS_COMPRESSED_ROW_PADDING_DIRECT, (int64_t)sub, e);
        as_execute_strategy(m, AS_COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE, (int64_t)sub, none);
        as_complete_blocking(m, (int64_t)sub);
      }
      as_builder *b = as_builder_create(m);
      bool set = true;
      for (uint64_t sub = 0; sub < info[4]; sub++) set = set && as_builder_set_template(b, (int64_t)sub, AS_DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS) == 0;
      if (set && as_builder_kernel_source(b)) built++;
      as_builder_free(b);
      as_matrix_free(m);
      (void)d;
    }
    printf("case %d (law %d, %llu rows, %zu elements): built %d so far, %d api errors\n", cs, law, (unsigned long long)c.rows, c.r.size(), built, fails);
    fflush(stdout);
  }
  printf("done: %d kernels' sources built, %d api errors\n", built, fails);
  return 0;
}
