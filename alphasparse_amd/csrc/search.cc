#include "search.hpp"
#include "graph_enumerate.hpp"

#include <array>
#include <cmath>
#include <cstdio>
#include <fstream>
#include <map>

#include "device_facts.hpp"
#include "hip_layer.h"

namespace asx {

// ---------------------------------------------------------------------------------------------
MatrixInfo get_matrix_info(const Matrix &m) {
  MatrixInfo i;
  i.row_nnz = get_nnz_of_each_row(m);
  i.nnz = m.nnz; i.row_num = m.rows; i.col_num = m.cols; i.is_sorted = m.is_sorted;
  i.is_double = m.val_dtype == DOUBLE;
  i.max_row_nnz = *std::max_element(i.row_nnz.begin(), i.row_nnz.end());
  i.min_row_nnz = *std::min_element(i.row_nnz.begin(), i.row_nnz.end());
  i.avg_row_nnz = i.nnz / i.row_num;
  return i;
}

MatrixInfo get_sub_matrix_info_from_compressed_matrix_block(const Matrix &m, uint64_t sub) {
  AS_CHECK(sub < m.items.size() && m.items[sub].cb, "sub-matrix is not compressed");
  MatrixInfo i;
  i.row_nnz = get_nnz_of_each_row_in_compressed_sub_matrix(*m.items[sub].cb);
  i.nnz = m.items[sub].cb->read_index[0]->length;
  i.row_num = i.row_nnz.size();
  i.col_num = m.items[sub].max_col - m.items[sub].min_col + 1;
  i.is_sorted = m.is_sorted;
  i.is_double = m.val_dtype == DOUBLE;
  i.max_row_nnz = *std::max_element(i.row_nnz.begin(), i.row_nnz.end());
  i.min_row_nnz = *std::min_element(i.row_nnz.begin(), i.row_nnz.end());
  i.avg_row_nnz = i.nnz / i.row_num;
  // blocks of rows with the same columns, judged from the first 48 rows (elements are still row by row here)
  if (m.items[sub].cb->read_index.size() == 2) {
    const std::vector<uint64_t> &col = m.items[sub].cb->read_index[1]->index_arr.v;
    std::vector<uint64_t> start{0};
    for (uint64_t r = 0; r < std::min<uint64_t>(i.row_num, 48); r++) start.push_back(start.back() + i.row_nnz[r]);
    const uint64_t rows = start.size() - 1;
    for (uint64_t h : {4, 3, 2}) {
      if (i.row_num % h != 0 || rows < 2 * h) continue;
      bool same = true;
      for (uint64_t blk = 0; same && blk < rows / h; blk++)
        for (uint64_t q = 1; same && q < h; q++) {
          const uint64_t a = start[blk * h], b = start[blk * h + q], len = start[blk * h + 1] - a;
          same = start[blk * h + q + 1] - b == len;
          for (uint64_t e = 0; same && e < len; e++) same = col[a + e] == col[b + e];
        }
      if (same) { i.row_block = h; break; }
    }
    // distinct diagonals, where a row is short enough for the ELL template to be in question at all
    if (i.max_row_nnz <= 64) {
      const std::vector<uint64_t> &row = m.items[sub].cb->read_index[0]->index_arr.v;
      std::vector<int64_t> seen;
      int64_t last = INT64_MIN;
      for (size_t k = 0; k < col.size() && seen.size() <= 64; k++) {
        const int64_t d = (int64_t)col[k] - (int64_t)row[k];
        if (d == last) continue;
        last = d;
        if (std::find(seen.begin(), seen.end(), d) == seen.end()) seen.push_back(d);
      }
      i.diagonals = seen.size();
    }
  }
  return i;
}

// ---------------------------------------------------------------------------------------------
void ParamEnumerator::add(long *ptr, long low, long up, long step) {
  AS_CHECK(ptr && low <= up && step >= 1, "bad knob range");
  for (auto &k : knobs) AS_CHECK(k.ptr != ptr, "knob registered twice");
  *ptr = low - 1;  // upstream: a knob rests one below its range until the first advance
  knobs.push_back({ptr, low, up, step});
}

bool ParamEnumerator::next() {
  AS_CHECK(!knobs.empty(), "no knob registered");
  for (;;) {
    if (!started) {
      for (auto &k : knobs) *k.ptr = k.low;
      started = true;
    } else {
      size_t i = 0;
      for (; i < knobs.size(); i++) {
        Knob &k = knobs[i];
        if (*k.ptr + k.step <= k.up) { *k.ptr += k.step; break; }
        *k.ptr = k.low;  // wrap and carry into the next knob
      }
      if (i == knobs.size()) return false;
    }
    bool ok = true;
    for (auto &f : filters) ok = ok && f();
    if (ok) return true;
  }
}

// ---------------------------------------------------------------------------------------------
SearchStrategy init_search_strategy(uint64_t struggle, double total) {
  SearchStrategy s;
  s.remain_step_num = 10;
  s.struggle_step_num = struggle;
  s.total_allow_search_time = total;
  s.begin_time = std::chrono::steady_clock::now();
  return s;
}
static double elapsed(const SearchStrategy &s) {
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - s.begin_time).count();
}
bool continue_search(SearchStrategy &s, float gflops) {
  if (gflops > s.best_glops) {
    // window of further trials after an improvement: 5 per GFLOP/s gained, within [5, 25]
    double w = (double)(gflops - s.best_glops) * 5.0;
    s.remain_step_num = (uint64_t)std::min(25.0, std::max(5.0, std::floor(w)));
    s.best_glops = gflops;
  } else if (s.remain_step_num > 0) s.remain_step_num--;
  else if (s.struggle_step_num > 0) s.struggle_step_num--;
  else return false;
  return elapsed(s) < s.total_allow_search_time;
}
bool continue_search(const SearchStrategy &s) {
  if (elapsed(s) >= s.total_allow_search_time) return false;
  return !(s.remain_step_num == 0 && s.struggle_step_num == 0);
}

// ---------------------------------------------------------------------------------------------
std::string convert_template_node_to_string(const TemplateNode &n) {
  auto res = [&](bool with_grid) {
    std::string s = "kernel_node_type:SET_RESOURCE\n{\nthread_num_in_block:" + std::to_string(n.thread_num_in_block) + "\n";
    if (with_grid) s += "tblock_num:" + std::to_string(n.tblock_num) + "\n";
    if (n.col_relative == 1) s += "col_index_relative:1\n";  // not upstream keys
    if (n.col_relative == 2) s += "col_index_diagonal:1\n";
    if (n.col_relative == 3) s += "col_index_runs:1\n";
    if (n.own_rows == 1) s += "y_rows_owned:1\n";
    if (n.row_block > 1) s += "row_block:" + std::to_string(n.row_block) + "\n";
    // upstream closes every kernel node with one more "}" than it opened (exe_graph.cc:3547); kept,
    // since readers of test.log are written against that text
    return s + "}\n}\n";
  };
  auto red = [&](const char *first) {
    return std::string("kernel_node_type:") + first + "\nkernel_node_type:SHARED_MEM_OFFSET_RED\n{\nthread_num_of_row_reduce:" +
           std::to_string(n.thread_num_of_row_reduce) + "\nhybrid_reduce:0\n}\n";
  };
  switch (n.type) {
    case DIRECT_ATOM_TEMPLATE:
    case DIRECT_ATOM_TEMPLATE_WARP_COMPRESS:
    case DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS:
      return "kernel_node_type:THREAD_TOTAL_RED\nkernel_node_type:GBL_ATOM_RED\n" + res(true);
    case SHARED_MEMORY_TEMPLATE:
    case SHARED_MEMORY_TEMPLATE_WARP_COMPRESS:
      return red("THREAD_TOTAL_RED") + res(true);
    case SHARED_MEMORY_LONG_ROW_TEMPLATE:
      return "kernel_node_type:SHARED_MEM_TOTAL_RED\nkernel_node_type:GBL_ATOM_RED\n" + res(true);
    case SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE:
      return red("WARP_TOTAL_RED") + res(true);
    case DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE:
      return "kernel_node_type:WARP_TOTAL_RED\nkernel_node_type:GBL_ATOM_RED\n" + res(true);
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE:
      return "kernel_node_type:THREAD_BITMAP_RED\nkernel_node_type:WARP_SEG_ADD_RED\n{\nhybrid_reduce:0\n}\n" + res(true);
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE:
      return "kernel_node_type:THREAD_BITMAP_RED\nkernel_node_type:WARP_SEG_ADD_RED\n{\nhybrid_reduce:1\n}\n" + res(false);
    case SHARED_MEMORY_X_SLICE_TEMPLATE:  // no upstream counterpart
      return "kernel_node_type:SHARED_MEM_X_SLICE\nkernel_node_type:WARP_TOTAL_RED\nkernel_node_type:GBL_ATOM_RED\n" + res(true);
    case SHARED_MEMORY_PRODUCT_BIN_TEMPLATE:  // no upstream counterpart
      return "kernel_node_type:SHARED_MEM_X_SLICE\nkernel_node_type:GBL_PRODUCT_BIN\nkernel_node_type:WARP_SEG_ADD_RED\n"
             "kernel_node_type:SHARED_MEM_TOTAL_RED\n" + res(true);
    case SHARED_MEMORY_TILE_TEMPLATE:  // no upstream counterpart
      return "kernel_node_type:SHARED_MEM_X_SLICE\nkernel_node_type:WARP_SEG_ADD_RED\nkernel_node_type:SHARED_MEM_TOTAL_RED\n"
             "kernel_node_type:GBL_ATOM_RED\n" + res(true);
    default:
      throw Error("convert_template_node_to_string: template type is not supported");
  }
}

std::string convert_graph_to_string(const BestGraph &g) {
  std::string s = convert_all_stategy_node_of_sub_matrix_to_string(g.dense);
  for (size_t i = 0; i < g.subs.size(); i++) {
    s += "sub_matrix_id:" + std::to_string(i) + "\n";
    s += convert_all_stategy_node_of_sub_matrix_to_string(g.subs[i].nodes);
    s += convert_template_node_to_string(g.subs[i].tpl);
  }
  return s;
}

// What upstream's main prints once the search is over (main.cc:646-657): the two figures, the graph followed by an
// empty line (the string already ends its last line, `<< endl` adds another), or "error" when nothing ran, then
// "finish search".
std::string convert_search_result_to_string(float gflops, float time_ms, const BestGraph &g) {
  char head[256];
  snprintf(head, sizeof head, "gflops:%g\ntime:%g\n", gflops, time_ms);
  return std::string(head) + (gflops != 0 ? convert_graph_to_string(g) + "\n" : std::string("error\n")) + "finish search\n";
}

// ---------------------------------------------------------------------------------------------
namespace {

struct Ctx {
  const SearchOptions &opt;
  SearchResult &res;
  SearchStrategy global;
  // the vector every candidate is checked (and timed) with, in the value type, `cols` entries: x[j] = 1 + j % 7.
  // Not constant on purpose: a kernel that reads x at a wrong place (relative, diagonal and column-run column
  // forms, x-slice offsets, the first column of a column band) gives a wrong y with it, which x = 1 would hide
  std::vector<uint8_t> probe_x;
  bool empty_rows = false;    // the input has rows without elements and they are removed first
  // per row of the input: y for that x (a host CSR product computed once per search), and the same sum over the
  // magnitudes
  std::vector<double> row_sum, row_mag;
  std::vector<uint64_t> row_len;   // elements of every row of the input
  // time per SpMV (ms) of the best whole graph measured so far, 0 before the first: a strip kernel that alone takes
  // longer cannot be part of a better graph, whichever way the strips are launched
  float best_whole_ms = 0;
  std::chrono::steady_clock::time_point t0 = std::chrono::steady_clock::now();
  // " @12.3s": seconds since the search began, appended to the lines that open a phase
  double now_s() const { return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count(); }
  std::string stamp() const {
    char b[32];
    snprintf(b, sizeof b, " @%.1fs", now_s());
    return b;
  }
  void log(const std::string &line) {
    res.log += line + "\n";
    if (opt.verbose) { fputs((line + "\n").c_str(), stderr); }
  }
};

void set_launch(Template &t, const TemplateNode &n) {
  t.vec_width = (unsigned)n.vec_width;
  t.thread_num_in_block = (uint64_t)n.thread_num_in_block;
  if (n.thread_num_of_row_reduce > 0) t.thread_num_of_row_reduce = (uint64_t)n.thread_num_of_row_reduce;
  set_default_launch(t);
  if (n.tblock_num > 0) t.tblock_num = (uint64_t)n.tblock_num;
}

// One SpMV with the search's probe vector (x[j] = 1 + j % 7): the rows that the loaded kernels cover (sub-matrix
// `sub`, or all with sub < 0) must hold the host's product for that x, every other row of y zero.  Throws on a
// mismatch.
void verify_candidate(Ctx &c, Builder &b, const Matrix &m, int64_t sub) {
  if (!c.opt.verify_candidates) return;
  launch_spmv(b, b.x.ptr, b.y.ptr);
  if (as_hip_stream_sync(b.main_stream) != 0) throw Error(as_hip_last_error());
  const bool f64 = b.val_dtype == DOUBLE;
  std::vector<uint8_t> y(b.y.bytes);
  if (as_hip_d2h(y.data(), b.y.ptr, b.y.bytes) != 0) throw Error(as_hip_last_error());
  AS_CHECK(b.rows == c.row_sum.size(), "y and the input disagree on the number of rows");
  std::vector<uint8_t> covered(b.rows, sub < 0 ? 1 : 0);
  if (sub >= 0) {
    const DenseItem &it = m.items[(size_t)sub];
    for (uint64_t r = it.min_row; r <= it.max_row; r++) covered[m.sorted_row_index.present ? m.sorted_row_index[r] : r] = 1;
  }
  // 64 roundings of the value type on the sum of the magnitudes, times the row's length up to 16 (sums of long
  // rows are added up in trees and by atomics in any order): an element of a short row that is lost, doubled or
  // added to another row is far outside, and so is a typical element of a row of thousands
  const double eps64 = 64.0 * (f64 ? 2.220446049250313e-16 : 1.1920928955078125e-07);
  for (uint64_t r = 0; r < b.rows; r++) {
    const double got = f64 ? ((const double *)y.data())[r] : (double)((const float *)y.data())[r];
    const double want = covered[r] ? c.row_sum[r] : 0.0;
    const double tol = eps64 * (double)std::min<uint64_t>(16, std::max<uint64_t>(1, c.row_len[r]));
    if (!(std::fabs(got - want) <= tol * c.row_mag[r] + 1e-30))
      throw Error("wrong result: y[" + std::to_string(r) + "] = " + std::to_string(got) + " for a row sum of " +
                  std::to_string(want));
  }
}

bool time_builder(Ctx &c, Builder &b, float &ms_per_launch, float &gflops) {
  float ms = 0, gf = 0;
  time_spmv(b, 2, false, ms, gf);
  time_spmv(b, 3, false, ms, gf);
  double per = std::max(1e-4, (double)ms / 3.0);
  uint64_t reps = (uint64_t)std::min(2000.0, std::max(5.0, c.opt.timed_region_ms / per));
  time_spmv(b, reps, false, ms, gf);
  ms_per_launch = ms / (float)reps;
  gflops = gf;
  return true;
}

// launch-parameter sweeps per template family (default_auto_tuner.cc:449-2032, ranges set for
// 64-lane waves, <= 1024 threads per workgroup and 1/2/4-wide loads)
std::vector<TemplateNode> launch_candidates(const Template &t) {
  std::vector<TemplateNode> out;
  auto push = [&](long threads, long R, long vec) {
    TemplateNode n;
    n.type = t.type; n.thread_num_in_block = threads; n.thread_num_of_row_reduce = R; n.vec_width = vec;
    out.push_back(n);
  };
  auto round64 = [](uint64_t v) { return (long)std::min<uint64_t>(1024, std::max<uint64_t>(64, (v + 63) / 64 * 64)); };
  switch (t.type) {
    case DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS:
      for (long vec : {1, 2, 4})
        for (long th : {64, 128, 256}) push(th, 1, vec);
      break;
    case DIRECT_ATOM_TEMPLATE_WARP_COMPRESS: {
      uint64_t mx = t.sc("max_TLB_num_in_block");
      for (long vec : {1, 2, 4}) {
        long full = round64((mx + vec - 1) / vec);
        push(full, 1, vec);
        if (full >= 128) push(round64(full / 2), 1, vec);
      }
      break;
    }
    case DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE:
      for (long vec : {1, 2, 4})
        for (long th : {64, 256, 512}) push(th, 1, vec);
      break;
    case SHARED_MEMORY_LONG_ROW_TEMPLATE: {
      uint64_t mx = t.sc("max_BLB_nnz");
      for (long th : {64, 128, 256, 512, 1024})
        if ((uint64_t)th * 4 <= std::max<uint64_t>(256, mx)) push(th, 1, 4);
      break;
    }
    case SHARED_MEMORY_TEMPLATE_WARP_COMPRESS: {
      long full = round64(t.sc("max_TLB_num_in_block"));
      for (long R : {1, 4, 16}) {
        push(full, R, 1);
        if (full >= 256) push(round64(full / 2), R, 1);
      }
      break;
    }
    case SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE: {
      long full = round64(t.sc("max_WLB_num_in_block") * 64);
      for (long R : {1, 4, 16, 64})
        for (long vec : {1, 2}) {
          push(full, R, vec);
          if (full >= 256) push(round64(full / 2), R, vec);
        }
      break;
    }
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE:
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE:
      for (long th : {64, 128, 256}) push(th, 1, 1);
      break;
    case SHARED_MEMORY_X_SLICE_TEMPLATE:
      for (long th : {1024, 512}) push(th, 1, 1);
      break;
    case SHARED_MEMORY_TILE_TEMPLATE:
      for (long th : {1024, 512}) push(th, 1, 1);
      break;
    case SHARED_MEMORY_PRODUCT_BIN_TEMPLATE:
      for (long th : {1024, 512}) push(th, 1, 1);
      break;
    default:
      push(256, 1, 1);
  }
  return out;
}

// find_best_template_node_of_specific_sub_matrix_from_template_set (default_auto_tuner.cc:44):
// best (template, launch parameters) for an already built format of one sub-matrix
bool find_best_template(Ctx &c, Matrix &m, uint64_t sub, const std::vector<TemplateType> &types, SearchStrategy *local,
                        TemplateNode &best, float &best_gflops, float &best_ms, const MatrixInfo *info = nullptr,
                        uint64_t *best_bytes = nullptr) {
  best_gflops = 0;
  best_ms = 0;
  // useful bytes the best kernel so far moves per launch: its format arrays (scratch written and read included), x
  // once and the strip's rows of y once -- noted whenever `best` changes
  float noted_ms = -1;
  auto note_bytes = [&](const Builder &b) {
    if (!best_bytes || best_ms == noted_ms || !b.subs[sub].tpl) return;
    const uint64_t vs = (uint64_t)dtype_size(m.val_dtype);
    const uint64_t strip_rows = m.items[sub].max_row - m.items[sub].min_row + 1;
    const uint64_t format = template_format_bytes(*b.subs[sub].tpl) + m.cols * vs + strip_rows * vs;
    // ... but no more than a CSR of the strip with 32-bit columns would move: padding is not useful work
    const uint64_t csr = b.subs[sub].tpl->origin_nnz * (vs + 4) + (strip_rows + 1) * 4 + (m.cols + strip_rows) * vs;
    *best_bytes = std::min(format, csr);
    noted_ms = best_ms;
  };
  execute_default_div_to_complete_each_level_blocking(m, sub);
  const CompressedBlock &cb = *m.items[sub].cb;
  double rate = (double)cb.padding_val->size() / (double)cb.read_index[0]->length;
  if (rate > c.opt.padding_rate_up_bound) {
    c.log("  padding rate " + std::to_string(rate) + " above the bound, candidate skipped");
    return false;
  }
  for (TemplateType type : types) {
    if (!is_supported_by_template(type, m, sub)) continue;
    std::unique_ptr<Builder> b;
    // A stencil (as many diagonals as the longest row has elements) through the ELL template: the form without a
    // column array first, and the launch settings swept in that form -- it is what wins there, and the sooner it is
    // measured the sooner a caller has its graph.
    long first_form = 0;
    // A banded matrix whose rows come in blocks with the same columns through the tile template: the form that has
    // won on such matrices (column runs where they shorten the stream, row ownership, blocks of rows as pieces) is
    // built and measured first; the plain form and the steps towards it follow only where it does not apply.
    bool tile_blocks_first = false;
    try {
      b = init_code_builder(m);
      if (type == SHARED_MEMORY_TILE_TEMPLATE && info && info->row_block > 1 && is_supported_by_template(type, m, sub) &&
          add_tile_template_variant_to_builder(*b, sub, true, true, info->row_block)) {
        tile_blocks_first = true;
      } else {
        add_template_to_builder(*b, sub, type);
        compress_template_in_builder(*b, sub);
        if (type == DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS && info && info->diagonals > 0 &&
            info->diagonals <= std::max<uint64_t>(1, info->max_row_nnz) && set_diagonal_columns(*b, sub))
          first_form = 2;
      }
      load_and_upload(*b, c.opt.device);
      if (as_hip_h2d(b->x.ptr, c.probe_x.data(), b->x.bytes) != 0) throw Error(as_hip_last_error());
    } catch (const std::exception &e) {
      c.res.failed_candidates++;
      c.log(std::string("  candidate failed: ") + e.what());
      continue;
    }
    if (tile_blocks_first) {
      bool measured = false;
      for (long threads : {1024l, 512l}) {
        TemplateNode n;
        n.type = type; n.thread_num_in_block = threads; n.thread_num_of_row_reduce = 1; n.vec_width = 1;
        n.col_relative = b->subs[sub].tpl->col_runs ? 3 : 0;
        n.own_rows = 1;
        n.row_block = (long)info->row_block;
        float ms = 0, gf = 0;
        try {
          set_launch(*b->subs[sub].tpl, n);
          invalidate_module(*b);
          verify_candidate(c, *b, m, (int64_t)sub);
          time_builder(c, *b, ms, gf);
        } catch (const std::exception &e) {
          c.res.failed_candidates++;
          c.log(std::string("  candidate failed: ") + e.what());
          continue;
        }
        c.res.candidates++;
        measured = true;
        n.tblock_num = (long)b->subs[sub].tpl->tblock_num;
        c.log(std::string("  template sub_matrix_id:") + std::to_string(sub) + " " + convert_template_type_to_string(type) +
              " threads " + std::to_string(n.thread_num_in_block) + " blocks " + std::to_string(n.tblock_num) +
              (n.col_relative == 3 ? " column runs," : "") + " row ownership, row blocks of " + std::to_string(n.row_block) +
              " -> " + std::to_string(gf) + " GFLOP/s, " + std::to_string(ms * 1e3f) + " us" + c.stamp());
        if (gf > best_gflops * (best_gflops > 0 && best.type == type ? 1.01f : 1.0f)) { best_gflops = gf; best_ms = ms; best = n; note_bytes(*b); }
        bool go = local ? continue_search(*local, gf) : true;
        if (!go || !continue_search(c.global)) return best_gflops > 0;
      }
      if (measured) continue;   // the other forms of the tile template are steps towards this one
      // it did not run: the plain form and its refinements below
      try {
        add_template_to_builder(*b, sub, type);
        compress_template_in_builder(*b, sub);
        load_and_upload(*b, c.opt.device);
      } catch (const std::exception &e) {
        c.res.failed_candidates++;
        c.log(std::string("  candidate failed: ") + e.what());
        continue;
      }
    }
    for (TemplateNode n : launch_candidates(*b->subs[sub].tpl)) {
      float ms = 0, gf = 0;
      n.col_relative = first_form;
      try {
        set_launch(*b->subs[sub].tpl, n);
        invalidate_module(*b);
        verify_candidate(c, *b, m, (int64_t)sub);
        time_builder(c, *b, ms, gf);
      } catch (const std::exception &e) {
        c.res.failed_candidates++;
        c.log(std::string("  candidate failed: ") + e.what());
        continue;
      }
      c.res.candidates++;
      n.tblock_num = (long)b->subs[sub].tpl->tblock_num;
      n.thread_num_in_block = (long)b->subs[sub].tpl->thread_num_in_block;
      c.log(std::string("  template sub_matrix_id:") + std::to_string(sub) + " " + convert_template_type_to_string(type) +
            " threads " + std::to_string(n.thread_num_in_block) + " blocks " + std::to_string(n.tblock_num) + " row_reduce " +
            std::to_string(n.thread_num_of_row_reduce) + " vec " + std::to_string(n.vec_width) + " -> " + std::to_string(gf) +
            (first_form == 2 ? " diagonal columns" : "") + " GFLOP/s, " + std::to_string(ms * 1e3f) + " us");
      // another launch setting of the template that leads must lead by more than the noise of two timings (1 %):
      // the same matrix then gets the same graph from one search to the next
      const bool same_template = best_gflops > 0 && best.type == type;
      if (gf > best_gflops * (same_template ? 1.01f : 1.0f)) { best_gflops = gf; best_ms = ms; best = n; note_bytes(*b); }
      bool go = local ? continue_search(*local, gf) : true;
      if (!go || !continue_search(c.global)) return best_gflops > 0;
      // launch settings of one format differ by tens of percent, not by factors: a format whose first setting alone
      // takes more than twice the best whole SpMV so far is not swept
      if (c.best_whole_ms > 0 && ms > 2.0f * c.best_whole_ms) {
        c.log("  first launch setting alone takes more than 2 x the best whole SpMV so far, other settings skipped");
        break;
      }
    }
    // the best launch of the ELL template once more with 16-bit relative columns and then with the columns
    // computed from the slots' diagonals, where the matrix allows them
    if (type == DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS && first_form == 0 && best.type == type && best_gflops > 0) {
      const TemplateNode launch = best;
      for (long form : {1l, 2l}) {
        try {
          if (!(form == 1 ? set_relative_columns(*b, sub) : set_diagonal_columns(*b, sub))) continue;
          load_and_upload(*b, c.opt.device);
          TemplateNode n = launch;
          n.col_relative = form;
          set_launch(*b->subs[sub].tpl, n);
          invalidate_module(*b);
          verify_candidate(c, *b, m, (int64_t)sub);
          float ms = 0, gf = 0;
          time_builder(c, *b, ms, gf);
          c.res.candidates++;
          c.log(std::string("  template sub_matrix_id:") + std::to_string(sub) + " " + convert_template_type_to_string(type) +
                " threads " + std::to_string(n.thread_num_in_block) + " vec " + std::to_string(n.vec_width) +
                (form == 1 ? " relative columns -> " : " diagonal columns -> ") + std::to_string(gf) + " GFLOP/s, " +
                std::to_string(ms * 1e3f) + " us");
          if (gf > best_gflops) { best_gflops = gf; best_ms = ms; best = n; note_bytes(*b); }
        } catch (const std::exception &e) {
          c.res.failed_candidates++;
          c.log(std::string("  candidate failed: ") + e.what());
        }
      }
    }
    // the best launch of the tile template once more in its column-run form, where that shortens the stream
    if (type == SHARED_MEMORY_TILE_TEMPLATE && best.type == type && best_gflops > 0) {
      try {
        if (set_column_runs(*b, sub)) {
          load_and_upload(*b, c.opt.device);
          TemplateNode n = best;
          n.col_relative = 3;
          set_launch(*b->subs[sub].tpl, n);
          invalidate_module(*b);
          verify_candidate(c, *b, m, (int64_t)sub);
          float ms = 0, gf = 0;
          time_builder(c, *b, ms, gf);
          c.res.candidates++;
          n.tblock_num = (long)b->subs[sub].tpl->tblock_num;
          c.log(std::string("  template sub_matrix_id:") + std::to_string(sub) + " " + convert_template_type_to_string(type) +
                " threads " + std::to_string(n.thread_num_in_block) + " blocks " + std::to_string(n.tblock_num) +
                " column runs -> " + std::to_string(gf) + " GFLOP/s, " + std::to_string(ms * 1e3f) + " us");
          if (gf > best_gflops) { best_gflops = gf; best_ms = ms; best = n; note_bytes(*b); }
        }
      } catch (const std::exception &e) {
        c.res.failed_candidates++;
        c.log(std::string("  candidate failed: ") + e.what());
      }
      // and the best of the two once more under row ownership (whole row groups per workgroup, rows stored
      // without atomics, no clear of y), where the sub-matrix allows it
      try {
        add_template_to_builder(*b, sub, type);
        compress_template_in_builder(*b, sub);
        if (best.col_relative == 3) AS_CHECK(set_column_runs(*b, sub), "column runs cannot be rebuilt");
        if (set_row_ownership(*b, sub)) {
          load_and_upload(*b, c.opt.device);
          if (as_hip_h2d(b->x.ptr, c.probe_x.data(), b->x.bytes) != 0) throw Error(as_hip_last_error());
          TemplateNode n = best;
          n.own_rows = 1;
          n.tblock_num = 0;  // one workgroup per trip of the new form
          set_launch(*b->subs[sub].tpl, n);
          invalidate_module(*b);
          verify_candidate(c, *b, m, (int64_t)sub);
          float ms = 0, gf = 0;
          time_builder(c, *b, ms, gf);
          c.res.candidates++;
          n.tblock_num = (long)b->subs[sub].tpl->tblock_num;
          c.log(std::string("  template sub_matrix_id:") + std::to_string(sub) + " " + convert_template_type_to_string(type) +
                " threads " + std::to_string(n.thread_num_in_block) + " blocks " + std::to_string(n.tblock_num) +
                " row ownership -> " + std::to_string(gf) + " GFLOP/s, " + std::to_string(ms * 1e3f) + " us");
          if (gf > best_gflops) { best_gflops = gf; best_ms = ms; best = n; note_bytes(*b); }
          // and, where the rows come in blocks that hold the same columns, with a block of rows as one piece
          const uint64_t height = best.own_rows == 1 ? tile_row_block_guess(m, sub) : 1;
          if (height > 1 && set_row_blocks(*b, sub, height)) {
            load_and_upload(*b, c.opt.device);
            if (as_hip_h2d(b->x.ptr, c.probe_x.data(), b->x.bytes) != 0) throw Error(as_hip_last_error());
            n.row_block = (long)height;
            n.tblock_num = 0;
            set_launch(*b->subs[sub].tpl, n);
            invalidate_module(*b);
            verify_candidate(c, *b, m, (int64_t)sub);
            time_builder(c, *b, ms, gf);
            c.res.candidates++;
            n.tblock_num = (long)b->subs[sub].tpl->tblock_num;
            c.log(std::string("  template sub_matrix_id:") + std::to_string(sub) + " " + convert_template_type_to_string(type) +
                  " threads " + std::to_string(n.thread_num_in_block) + " blocks " + std::to_string(n.tblock_num) +
                  " row blocks of " + std::to_string(height) + " -> " + std::to_string(gf) + " GFLOP/s, " + std::to_string(ms * 1e3f) + " us");
            if (gf > best_gflops) { best_gflops = gf; best_ms = ms; best = n; note_bytes(*b); }
          }
        }
      } catch (const std::exception &e) {
        c.res.failed_candidates++;
        c.log(std::string("  candidate failed: ") + e.what());
      }
    }
  }
  return best_gflops > 0;
}

struct Skeleton {
  const char *name;
  std::vector<TemplateType> templates;
  // knobs + how to turn them into strategy nodes
  std::function<void(ParamEnumerator &, long *)> knobs;
  std::function<std::vector<StrategyNode>(const long *)> nodes;
  // cheap estimate of padded elements / elements before the format is built (upstream
  // whilte_list_path_impl.cc:270-335); empty = no estimate
  std::function<double(const long *)> padding_estimate;
};

long ceil_to(long v, long m) { return (v + m - 1) / m * m; }

// The nine white-list skeletons (whilte_list_path_impl.cc:180-3095) with their gates (:3453-4034).
std::vector<Skeleton> skeletons_for(const MatrixInfo &info, bool globally_sorted, unsigned wave, bool general_templates) {
  std::vector<Skeleton> out;
  const long mn = (long)info.min_row_nnz, mx = (long)info.max_row_nnz, avg = (long)info.avg_row_nnz, W = (long)wave;
  auto S8 = [&]() {  // one-row BLBs of b elements, long-row kernel
    Skeleton s;
    s.name = "S8";
    s.templates = {SHARED_MEMORY_LONG_ROW_TEMPLATE};
    long hi = std::max(256l, ceil_to(mx, 256));
    s.knobs = [hi](ParamEnumerator &e, long *k) {
      // b = 256 << k0, at most up to the longest row
      long steps = 0;
      while ((256l << (steps + 1)) <= hi && steps < 6) steps++;
      e.add(&k[0], 0, steps, 1);
    };
    s.nodes = [](const long *k) {
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY, 256l << k[0])};
    };
    return s;
  };
  auto S1 = [&]() {  // SELL
    Skeleton s;
    s.name = "S1";
    s.templates = {DIRECT_ATOM_TEMPLATE_WARP_COMPRESS};
    s.knobs = [W](ParamEnumerator &e, long *k) { e.add(&k[0], 0, 3, 1); (void)W; };
    s.nodes = [W](const long *k) {
      long m = W << k[0];  // 64, 128, 256, 512 rows per BLB
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY, m, 1),
                                       make_strategy(COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY, m),
                                       make_strategy(COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY)};
    };
    const MatrixInfo *ip = &info;
    s.padding_estimate = [W, ip](const long *k) {
      uint64_t m = (uint64_t)(W << k[0]), padded = 0;
      for (uint64_t r0 = 0; r0 < ip->row_num; r0 += m) {
        uint64_t mxr = 1;
        for (uint64_t r = r0; r < std::min<uint64_t>(ip->row_num, r0 + m); r++) mxr = std::max(mxr, ip->row_nnz[r]);
        padded += mxr * m;
      }
      return (double)padded / (double)ip->nnz;
    };
    return s;
  };
  auto S5 = [&]() {  // ELL
    Skeleton s;
    s.name = "S5";
    s.templates = {DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS};
    s.knobs = [](ParamEnumerator &e, long *k) { e.add(&k[0], 0, 0, 1); };
    s.nodes = [W](const long *) {
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY, W, 1),
                                       make_strategy(COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY)};
    };
    const MatrixInfo *ip = &info;
    s.padding_estimate = [W, ip](const long *) {
      uint64_t rows = (ip->row_num + W - 1) / W * W;
      return (double)(rows * ip->max_row_nnz) / (double)ip->nnz;
    };
    return s;
  };
  auto S9 = [&]() {  // CSR5-like
    Skeleton s;
    s.name = "S9";
    s.templates = {UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE, UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE};
    long hi = std::min(32l, std::max(2l, avg)), step = std::max(1l, (hi - 2) / 4);
    s.knobs = [hi, step](ParamEnumerator &e, long *k) { e.add(&k[0], 2, hi, step); };
    s.nodes = [](const long *k) {
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT_PARAM_STRATEGY, k[0])};
    };
    return s;
  };
  auto S4 = [&]() {  // fixed-size row pieces, one wave each
    Skeleton s;
    s.name = "S4";
    s.templates = {DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE};
    long step = std::max(W, ceil_to((mx - mn + 2) / 3, W)), hi = std::max(W, ceil_to(mx, W));
    s.knobs = [W, step, hi](ParamEnumerator &e, long *k) { e.add(&k[0], W, std::max(W, hi), step); };
    s.nodes = [](const long *k) {
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY, k[0])};
    };
    return s;
  };
  auto S6 = [&]() {
    Skeleton s;
    s.name = "S6";
    s.templates = {SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE};
    long chi = std::max(W, std::min(2 * W, mx / 2 / W * W));
    s.knobs = [W, chi](ParamEnumerator &e, long *k) {
      e.add(&k[0], 2, 4, 2);      // rows per BLB
      e.add(&k[1], W, chi, W);    // elements per WLB
    };
    s.nodes = [mn](const long *k) {
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY, k[0], std::max(1l, mn)),
                                       make_strategy(COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY, k[0]),
                                       make_strategy(COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY, k[1])};
    };
    return s;
  };
  auto S7 = [&]() {
    Skeleton s;
    s.name = "S7";
    s.templates = {SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE};
    long chi = std::max(W, mx / 2 / W * W);
    s.knobs = [W, chi](ParamEnumerator &e, long *k) {
      e.add(&k[0], 0, 2, 1);                       // BLB nnz bound 512, 2048, 4096
      e.add(&k[1], W, std::min(chi, 4 * W), W);    // elements per WLB
    };
    s.nodes = [](const long *k) {
      static const long n[] = {512, 2048, 4096};
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY, n[k[0]]),
                                       make_strategy(COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY, k[1])};
    };
    return s;
  };
  auto S2 = [&]() {
    Skeleton s;
    s.name = "S2";
    s.templates = {SHARED_MEMORY_TEMPLATE_WARP_COMPRESS};
    long shi = std::max(1l, std::min(16l, (mx + 1) / 2));
    s.knobs = [W, shi](ParamEnumerator &e, long *k) {
      e.add(&k[0], 0, 1, 1);     // 64 or 128 rows per BLB
      e.add(&k[1], 1, shi, 3);   // TLB size
    };
    s.nodes = [W, mn](const long *k) {
      long m = W << k[0];
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY, m, std::max(1l, mn)),
                                       make_strategy(COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY, m),
                                       make_strategy(COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY, k[1])};
    };
    return s;
  };
  auto S3 = [&]() {
    Skeleton s;
    s.name = "S3";
    s.templates = {SHARED_MEMORY_TEMPLATE_WARP_COMPRESS};
    long shi = std::max(1l, std::min(16l, (mx + 1) / 2));
    s.knobs = [shi](ParamEnumerator &e, long *k) {
      e.add(&k[0], 0, 2, 1);
      e.add(&k[1], 1, shi, 3);
    };
    s.nodes = [](const long *k) {
      static const long n[] = {512, 2048, 4096};
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY, n[k[0]]),
                                       make_strategy(COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY, k[1])};
    };
    return s;
  };
  // one-row BLBs cut at column slice boundaries, x slice in LDS (no upstream counterpart).  Pays when
  // a row leaves enough elements in every slice it touches: shortest row / slices >= 32.
  auto S10 = [&]() {
    Skeleton s;
    s.name = "S10";
    s.templates = {SHARED_MEMORY_X_SLICE_TEMPLATE};
    long slice = (long)(x_slice_bytes() / (info.is_double ? 8 : 4));
    s.knobs = [](ParamEnumerator &e, long *k) { e.add(&k[0], 0, 0, 1); };
    s.nodes = [slice](const long *) {
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE_PARAM_STRATEGY, slice)};
    };
    return s;
  };
  // 2-D tiles: rows of one row group x columns of one slice, both staged in LDS (no upstream
  // counterpart).  Worth a try when x does not fit the L2 cache of an XCD and an average row leaves
  // an element in every fourth slice or more.  k0 = 0: one workgroup per CU (slice + row group fill the
  // 160 KB of LDS), 1: half-sized tiles, two workgroups per CU.
  auto S11 = [&]() {
    Skeleton s;
    s.name = "S11";
    s.templates = {SHARED_MEMORY_TILE_TEMPLATE};
    long slice = (long)(x_slice_bytes() / (info.is_double ? 8 : 4)), group = slice / 4;
    // rows that come in blocks of equal columns: row groups of whole blocks (halved groups too), so that the
    // template can store a block of rows as one piece
    if (info.row_block > 1) group = group / (2 * (long)info.row_block) * (2 * (long)info.row_block);
    s.knobs = [](ParamEnumerator &e, long *k) { e.add(&k[0], 0, 1, 1); };
    s.nodes = [slice, group](const long *k) {
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY,
                                                     slice >> k[0], group >> k[0], 8192)};
    };
    return s;
  };
  // the same elements in two passes (products streamed to scratch band by band of y, then summed band by band):
  // for rows too short to leave several elements per slice, where every x read of a row-wise kernel would
  // bring a cache line from HBM.  k0: slice width = 64, 128 or 32 KB of x (narrow slices: several first-pass
  // workgroups per CU, but shorter runs of products; C3: first pass 12.4 / 14.6 / 13.2 us, C5: 69.8 with 64 KB
  // against 66.0 with 128); k1: bands of 4096 or 2048 rows of y (C3: second pass 10.8 / 10.9 us, first pass
  // 13.2 / 14.7; 8192 rows: second pass 12.2).
  auto S12 = [&]() {
    Skeleton s;
    s.name = "S12";
    s.templates = {SHARED_MEMORY_PRODUCT_BIN_TEMPLATE};
    long slice = (long)(x_slice_bytes() / (info.is_double ? 8 : 4));
    s.knobs = [](ParamEnumerator &e, long *k) {
      e.add(&k[0], 0, 2, 1);
      e.add(&k[1], 0, 1, 1);
    };
    s.nodes = [slice](const long *k) {
      static const int shift[] = {1, 0, 2};
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY,
                                                     slice >> shift[k[0]], k[1] ? 2048 : 4096, 8192)};
    };
    return s;
  };
  // a stencil (no more diagonals than the longest row has elements): ELL first, its diagonal form is what wins
  const bool stencil = info.diagonals > 0 && info.diagonals <= (uint64_t)std::max(1l, mx);
  if (stencil && mx <= 512) out.push_back(S5());
  {
    long vs = info.is_double ? 8 : 4, slice = x_slice_bytes() / vs;
    long slices = ((long)info.col_num + slice - 1) / slice;
    if (slices >= 2 && (long)info.col_num * vs > (long)kL2BytesPerXcd && mx <= 64) out.push_back(S12());
    if (slices >= 2 && (long)info.col_num * vs > (long)kL2BytesPerXcd && avg >= std::max(8l, slices / 4)) out.push_back(S11());
    if (mn >= 32 * slices && slices >= 2) out.push_back(S10());
  }
  // The two general templates (outside upstream's white list; SearchOptions::general_templates): every
  // WLB has its own TLB size.  G1: BLBs of m rows, WLBs of w rows, one TLB per row, DIRECT_ATOM_TEMPLATE;
  // G2: BLBs by element count, WLBs of w rows, rows cut into TLBs of s elements, SHARED_MEMORY_TEMPLATE.
  auto G1 = [&]() {
    Skeleton s;
    s.name = "G1";
    s.templates = {DIRECT_ATOM_TEMPLATE};
    s.knobs = [](ParamEnumerator &e, long *k) {
      e.add(&k[0], 0, 2, 1);
      e.add(&k[1], 0, 1, 1);
    };
    s.nodes = [W](const long *k) {
      static const long m[] = {64, 256, 1024};
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY, m[k[0]]),
                                       make_strategy(COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY, k[1] ? W : W / 4),
                                       make_strategy(COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY)};
    };
    return s;
  };
  auto G2 = [&]() {
    Skeleton s;
    s.name = "G2";
    s.templates = {SHARED_MEMORY_TEMPLATE};
    long shi = std::max(1l, std::min(16l, (mx + 1) / 2));
    s.knobs = [shi](ParamEnumerator &e, long *k) {
      e.add(&k[0], 0, 1, 1);
      e.add(&k[1], 1, shi, 3);
    };
    s.nodes = [W](const long *k) {
      static const long n[] = {512, 4096};
      return std::vector<StrategyNode>{make_strategy(COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY, n[k[0]]),
                                       make_strategy(COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY, W / 4),
                                       make_strategy(COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY, k[1])};
    };
    return s;
  };
  if (general_templates && mx <= 512) { out.push_back(G1()); out.push_back(G2()); }
  // order tried upstream: 8, 1, 5, 9, 4, 6, 7, 2, 3
  if (mn >= 128) out.push_back(S8());
  if (mx <= 512) { out.push_back(S1()); if (!stencil) out.push_back(S5()); }
  if (!globally_sorted) out.push_back(S9());
  if (mn >= 30 && mx <= 512) out.push_back(S4());
  if (mn >= 32 && mx <= 1024) { out.push_back(S6()); out.push_back(S7()); }
  if (mx <= 1024) { out.push_back(S2()); out.push_back(S3()); }
  return out;
}

constexpr float kFamilyCutoff = 5.0f;
constexpr double kStreamingFrac = 0.62;
constexpr double kHbmPeakBytesPerSecond = 8e12;   // MI355X, HBM3E
constexpr float kWholeCutoff = 2.0f;

// find_best_path_of_compressed_sub_matrix (whilte_list_path_impl.cc:3411)
bool find_best_path_of_compressed_sub_matrix(Ctx &c, const Matrix &base, uint64_t sub, double budget_s, SubGraph &best) {
  MatrixInfo info = get_sub_matrix_info_from_compressed_matrix_block(base, sub);
  SearchStrategy local = init_search_strategy(c.opt.struggle_step_num, budget_s);
  best = SubGraph();
  c.log("sub_matrix_id:" + std::to_string(sub) + " rows " + std::to_string(info.row_num) + " nnz " + std::to_string(info.nnz) +
        " row nnz min/avg/max " + std::to_string(info.min_row_nnz) + "/" + std::to_string(info.avg_row_nnz) + "/" +
        std::to_string(info.max_row_nnz) + c.stamp());
  for (Skeleton &sk : skeletons_for(info, base.is_sorted, base.wave, c.opt.general_templates)) {
    long knob[4] = {0, 0, 0, 0};
    ParamEnumerator e;
    sk.knobs(e, knob);
    bool first_knob = true;
    while (e.next()) {
      std::vector<StrategyNode> nodes = sk.nodes(knob);
      std::string label = std::string(sk.name) + " knobs " + std::to_string(knob[0]) + "," + std::to_string(knob[1]);
      c.log(" " + label + c.stamp());
      if (sk.padding_estimate && sk.padding_estimate(knob) > c.opt.padding_rate_up_bound) {
        c.log("  estimated padding rate " + std::to_string(sk.padding_estimate(knob)) + " above the bound, graph skipped");
        continue;
      }
      std::unique_ptr<Matrix> m;
      try {
        m = base.clone_for_sub(sub);
        for (auto &n : nodes) {
          execute_param_strategy_node_of_sub_compressed_matrix(n, *m, sub);
          execute_exe_node_in_compressed_sub_matrix(*m, sub, n.node);
        }
      } catch (const std::exception &ex) {
        c.res.failed_candidates++;
        c.log(std::string("  graph rejected: ") + ex.what());
        continue;
      }
      TemplateNode tn;
      float gf = 0, ms = 0;
      uint64_t fmt_bytes = 0;
      bool ok = false;
      try {
        ok = find_best_template(c, *m, sub, sk.templates, &local, tn, gf, ms, &info, &fmt_bytes);
      } catch (const std::exception &ex) {
        c.res.failed_candidates++;
        c.log(std::string("  candidate failed: ") + ex.what());
      }
      if (ok && gf > best.gflops) {
        best.gflops = gf; best.time_ms = ms; best.tpl = tn;
        best.format_bytes = fmt_bytes;
        best.found_at_s = c.now_s();
        best.nodes = nodes;
        for (auto &n : best.nodes) n.node.reset_param();  // the graph keeps knobs, not expanded parameters
      }
      if (!continue_search(local) || !continue_search(c.global)) return best.gflops > 0;
      // A kernel that moves its format (+ x and the strip's rows of y; at most what a CSR of the strip would move) at
      // more than kStreamingFrac of the HBM peak is close to what a plain copy reaches on this device (0.75-0.78):
      // the skeletons and settings not tried yet could only win by a format of far fewer bytes, and the compact
      // formats are the ones in front.
      if (ok && best.time_ms > 0 && best.format_bytes > 0 &&
          (double)best.format_bytes / ((double)best.time_ms * 1e-3) > kStreamingFrac * kHbmPeakBytesPerSecond) {
        c.log("  the strip's kernel moves its format at more than " + std::to_string(kStreamingFrac) +
              " of the HBM peak: the remaining settings and skeletons are not tried" + c.stamp());
        return true;
      }
      // a family whose first setting runs at under a fifth of the strip's best is not swept further: its
      // settings differ among themselves by far less than that
      if (first_knob && ok && gf * kFamilyCutoff < best.gflops) {
        c.log("  " + std::string(sk.name) + ": first setting at under 1/" + std::to_string((int)kFamilyCutoff) +
              " of the strip's best, other settings skipped");
        break;
      }
      if (first_knob && ok && c.best_whole_ms > 0 && ms > kWholeCutoff * c.best_whole_ms) {
        c.log("  " + std::string(sk.name) + ": first setting alone takes more than " + std::to_string((int)kWholeCutoff) +
              " x the best whole SpMV so far, other settings skipped");
        break;
      }
      first_knob = false;
    }
  }
  return best.gflops > 0;
}

StrategyNode input_node(const CooInput &in) {
  StrategyNode n = make_strategy(DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY);
  n.in_nnz = in.row.size(); n.in_col_index_max = in.col_index_max; n.in_row_index_max = in.row_index_max;
  n.in_val_dtype = in.val_dtype;
  return n;
}

std::unique_ptr<Matrix> run_dense(const CooInput &in, std::vector<StrategyNode> &dense, unsigned wave, bool drop_empty_rows) {
  auto m = matrix_from_coo(in, wave);
  if (drop_empty_rows) remove_empty_rows(*m);
  for (auto &n : dense) {
    execute_param_strategy_node_of_dense_matrix(n, *m);
    execute_dense_node(*m, n.node);
  }
  return m;
}

// one dense-view strategy: per-strip search, then the combined graph is measured as a whole
bool search_dense_strategy(Ctx &c, const CooInput &in, std::vector<StrategyNode> dense, double budget_s, BestGraph &out) {
  std::unique_ptr<Matrix> base;
  try {
    base = run_dense(in, dense, c.opt.wave, c.empty_rows);
  } catch (const std::exception &e) {
    c.log(std::string("dense graph rejected: ") + e.what());
    return false;
  }
  size_t n_sub = base->items.size();
  if (n_sub > 4) { c.log("more than 4 strips, dense graph skipped"); return false; }
  out = BestGraph();
  out.dense = dense;
  out.empty_rows_removed = c.empty_rows;
  for (auto &n : out.dense) n.node.reset_param();
  out.subs.resize(n_sub);
  for (size_t s = 0; s < n_sub; s++) {
    // time per strip proportional to its nnz, within [1/2, 3] x the equal share (:4330-4577)
    double share = budget_s / (double)n_sub;
    double w = (double)(base->items[s].end_coo - base->items[s].begin_coo + 1) / (double)base->nnz * (double)n_sub;
    double t = share * std::min(3.0, std::max(0.5, w));
    if (!find_best_path_of_compressed_sub_matrix(c, *base, s, t, out.subs[s])) {
      c.log("no candidate for sub_matrix_id:" + std::to_string(s));
      return false;
    }
    if (n_sub > 1 && c.best_whole_ms > 0 && out.subs[s].time_ms > c.best_whole_ms) {
      c.log("sub_matrix_id:" + std::to_string(s) + " alone takes longer than the best whole SpMV so far, dense graph abandoned" + c.stamp());
      return false;
    }
  }
  if (n_sub == 1) {
    out.gflops = out.subs[0].gflops;
    out.time_ms = out.subs[0].time_ms;
    out.found_at_s = out.subs[0].found_at_s;
    if (c.best_whole_ms == 0 || out.time_ms < c.best_whole_ms) c.best_whole_ms = out.time_ms;
    return true;
  }
  try {
    BuiltGraph bg = build_from_graph(in, out, c.opt.wave);
    load_and_upload(*bg.builder, c.opt.device);
    if (as_hip_h2d(bg.builder->x.ptr, c.probe_x.data(), bg.builder->x.bytes) != 0) throw Error(as_hip_last_error());
    // Strip kernels that each take whole CUs (the LDS-tile templates: one or two workgroups fill a CU's LDS) only
    // get in each other's way on concurrent streams -- measured on every such graph so far (C3: 737 against 1042
    // GFLOP/s, C5: 540 against 632) -- so that way of launching is measured only where a strip has a kernel of
    // another kind.
    bool whole_cu_kernels = true;
    for (auto &sg : out.subs)
      whole_cu_kernels = whole_cu_kernels && (sg.tpl.type == SHARED_MEMORY_TILE_TEMPLATE || sg.tpl.type == SHARED_MEMORY_PRODUCT_BIN_TEMPLATE);
    if (!whole_cu_kernels) {
      verify_candidate(c, *bg.builder, *bg.matrix, -1);
      time_builder(c, *bg.builder, out.time_ms, out.gflops);
    }
    // kernels that each fill the machine can be faster one after the other than on concurrent streams
    float ms = 0, gf = 0;
    bg.builder->serial_launch = true;
    invalidate_module(*bg.builder);  // one after the other a finish kernel may be carried by the next strip's kernel
    verify_candidate(c, *bg.builder, *bg.matrix, -1);
    time_builder(c, *bg.builder, ms, gf);
    c.log("combined graph: " + (whole_cu_kernels ? std::string("not measured") : std::to_string(out.gflops) + " GFLOP/s") +
          " on concurrent streams, " + std::to_string(gf) + " GFLOP/s one after the other" + c.stamp());
    if (gf > out.gflops) { out.gflops = gf; out.time_ms = ms; out.serial_launch = true; }
    out.found_at_s = c.now_s();
    // A tile strip in front of a product-bin strip with workgroups of another size: with the same size in both, their
    // first kernels are one launch (Template::fused_trips).  Both common sizes are measured; the strips were tuned
    // one by one, the launch boundary between them is the whole graph's business.
    if (out.serial_launch)
      for (size_t i = 0; i + 1 < out.subs.size(); i++) {
        TemplateNode &tile = out.subs[i].tpl, &bin = out.subs[i + 1].tpl;
        if (tile.type != SHARED_MEMORY_TILE_TEMPLATE || bin.type != SHARED_MEMORY_PRODUCT_BIN_TEMPLATE ||
            tile.thread_num_in_block == bin.thread_num_in_block || assign_finish_carriers(*bg.builder, i) != (int64_t)(i + 1))
          continue;
        const long sizes[2] = {tile.thread_num_in_block, bin.thread_num_in_block};
        for (long threads : sizes) {
          TemplateNode t2 = tile, b2 = bin;
          t2.thread_num_in_block = b2.thread_num_in_block = threads;
          t2.tblock_num = b2.tblock_num = 0;
          try {
            set_launch(*bg.builder->subs[i].tpl, t2);
            set_launch(*bg.builder->subs[i + 1].tpl, b2);
            invalidate_module(*bg.builder);
            verify_candidate(c, *bg.builder, *bg.matrix, -1);
            time_builder(c, *bg.builder, ms, gf);
          } catch (const std::exception &e) {
            c.res.failed_candidates++;
            c.log(std::string("  candidate failed: ") + e.what());
            continue;
          }
          c.res.candidates++;
          c.log("combined graph, both strips with " + std::to_string(threads) + " threads (one launch for their first kernels): " +
                std::to_string(gf) + " GFLOP/s" + c.stamp());
          if (gf > out.gflops * 1.005f) {
            out.gflops = gf; out.time_ms = ms;
            t2.tblock_num = (long)bg.builder->subs[i].tpl->tblock_num;
            b2.tblock_num = (long)bg.builder->subs[i + 1].tpl->tblock_num;
            tile = t2; bin = b2;
            out.found_at_s = c.now_s();
          }
        }
        // leave the builder with the launch settings that won
        set_launch(*bg.builder->subs[i].tpl, tile);
        set_launch(*bg.builder->subs[i + 1].tpl, bin);
        invalidate_module(*bg.builder);
      }
  } catch (const std::exception &e) {
    c.log(std::string("combined graph failed: ") + e.what());
    return false;
  }
  if (c.best_whole_ms == 0 || out.time_ms < c.best_whole_ms) c.best_whole_ms = out.time_ms;
  return true;
}

}  // namespace

BuiltGraph build_from_graph(const CooInput &in, const BestGraph &g, unsigned wave) {
  BuiltGraph r;
  std::vector<StrategyNode> dense = g.dense;
  r.matrix = run_dense(in, dense, wave, g.empty_rows_removed);
  AS_CHECK(r.matrix->items.size() == g.subs.size(), "graph and matrix disagree on the number of sub-matrices");
  for (size_t s = 0; s < g.subs.size(); s++) {
    for (StrategyNode n : g.subs[s].nodes) {
      execute_param_strategy_node_of_sub_compressed_matrix(n, *r.matrix, s);
      execute_exe_node_in_compressed_sub_matrix(*r.matrix, s, n.node);
    }
    execute_default_div_to_complete_each_level_blocking(*r.matrix, s);
  }
  r.builder = init_code_builder(*r.matrix);
  r.builder->serial_launch = g.serial_launch;
  for (size_t s = 0; s < g.subs.size(); s++) {
    if (g.subs[s].tpl.type == SHARED_MEMORY_TILE_TEMPLATE && g.subs[s].tpl.own_rows == 1 && g.subs[s].tpl.row_block > 1) {
      // built at once, the way the search built it
      AS_CHECK(add_tile_template_variant_to_builder(*r.builder, s, g.subs[s].tpl.col_relative == 3, true, (uint64_t)g.subs[s].tpl.row_block) &&
                   r.builder->subs[s].tpl->col_runs == (g.subs[s].tpl.col_relative == 3),
               "the best graph's tile template cannot be rebuilt");
      set_launch(*r.builder->subs[s].tpl, g.subs[s].tpl);
      continue;
    }
    add_template_to_builder(*r.builder, s, g.subs[s].tpl.type);
    compress_template_in_builder(*r.builder, s);
    if (g.subs[s].tpl.col_relative == 1)
      AS_CHECK(set_relative_columns(*r.builder, s), "the best graph's relative columns cannot be rebuilt");
    if (g.subs[s].tpl.col_relative == 2)
      AS_CHECK(set_diagonal_columns(*r.builder, s), "the best graph's diagonal columns cannot be rebuilt");
    if (g.subs[s].tpl.col_relative == 3)
      AS_CHECK(set_column_runs(*r.builder, s), "the best graph's column runs cannot be rebuilt");
    if (g.subs[s].tpl.own_rows == 1)
      AS_CHECK(set_row_ownership(*r.builder, s), "the best graph's row ownership cannot be rebuilt");
    if (g.subs[s].tpl.row_block > 1)
      AS_CHECK(set_row_blocks(*r.builder, s, (uint64_t)g.subs[s].tpl.row_block), "the best graph's row blocks cannot be rebuilt");
    set_launch(*r.builder->subs[s].tpl, g.subs[s].tpl);
  }
  return r;
}

SearchResult find_best_graph_of_white_list_strategy(const CooInput &in, const SearchOptions &opt) {
  AS_CHECK(check_coo_sorted(in), "input must be sorted by (row, col)");
  const bool empty_rows = coo_has_empty_row(in);
  AS_CHECK(!empty_rows || opt.remove_empty_rows, "input must not have rows without elements");
  SearchResult res;
  Ctx c{opt, res, init_search_strategy(opt.struggle_step_num, opt.total_time_s), {}};
  // the formats are sized for the GPU the candidates run on
  if (as_hip_init(opt.device) != 0) throw Error(as_hip_last_error());
  read_device_facts(opt.device);
  c.empty_rows = empty_rows;
  if (empty_rows) c.log("rows without elements are removed before the first operator of every graph");
  size_t cols = in.col_index_max + 1;
  if (in.val_dtype == DOUBLE) {
    c.probe_x.resize(cols * 8);
    for (size_t i = 0; i < cols; i++) ((double *)c.probe_x.data())[i] = 1.0 + (double)(i % 7);
  } else {
    c.probe_x.resize(cols * 4);
    for (size_t i = 0; i < cols; i++) ((float *)c.probe_x.data())[i] = 1.0f + (float)(i % 7);
  }
  if (opt.verify_candidates) {
    c.row_sum.assign(in.row_index_max + 1, 0.0);
    c.row_mag.assign(in.row_index_max + 1, 0.0);
    c.row_len.assign(in.row_index_max + 1, 0);
    for (size_t i = 0; i < in.row.size(); i++) {
      const double xj = 1.0 + (double)(in.col[i] % 7);
      c.row_len[in.row[i]]++;
      c.row_sum[in.row[i]] += in.val[i] * xj;
      c.row_mag[in.row[i]] += std::fabs(in.val[i]) * xj;
    }
  }
  auto t_begin = std::chrono::steady_clock::now();
  auto now_s = [&]() { return std::chrono::duration<double>(std::chrono::steady_clock::now() - t_begin).count(); };
  std::vector<BestGraph> finalists;
  auto consider = [&](BestGraph &g, const char *name) {
    g.dense_strategy_name = name;
    c.log(std::string(name) + " best: " + std::to_string(g.gflops) + " GFLOP/s");
    if (!opt.checkpoint_dir.empty()) {
      // upstream keeps the best graph of each dense strategy in data_source/best_result_of_strategyN
      std::ofstream f(opt.checkpoint_dir + "/best_result_of_" + name);
      f << "gflops:" << g.gflops << "\ntime:" << g.time_ms << "\n" << convert_graph_to_string(g);
    }
    finalists.push_back(g);
    if (g.gflops > res.best.gflops) { res.best = g; res.seconds_to_best = g.found_at_s; }
  };
  StrategyNode input = input_node(in), compress = make_strategy(COMPRESS_NONE_PARAM_STRATEGY);
  const double T = opt.total_time_s;
  // strategies 2 and 3 cut the rows into bands of row length (0, low, low * rate, ... up to 2048, then
  // the rest).  When the shortest and the longest row fall into the same band for every (low, rate)
  // tried below, each of them yields one strip and is skipped (:4330+); strategy 1 then gets all the time.
  // row_len: the rows' lengths in row order (rows without elements left out: they are removed or the input was
  // rejected above); sorted_len: as the coarse sort with one bin per length leaves them, longest first.  The
  // strips of a row division follow from these without building the matrix.
  uint64_t longest_row = 0, shortest_row = ~0ull;
  std::vector<uint64_t> row_len;
  {
    uint64_t run = 0;
    for (size_t i = 0; i < in.row.size(); i++) {
      bool last_of_row = i + 1 == in.row.size() || in.row[i + 1] != in.row[i];
      run++;
      if (last_of_row) {
        longest_row = std::max(longest_row, run);
        shortest_row = std::min(shortest_row, run);
        row_len.push_back(run);
        run = 0;
      }
    }
  }
  std::vector<uint64_t> sorted_len = row_len;
  std::sort(sorted_len.begin(), sorted_len.end(), std::greater<uint64_t>());
  auto strips_of = [](const std::vector<uint64_t> &len, long low, long high, long rate) {
    std::vector<uint64_t> first = row_div_position_acc_to_exponential_increase_row_nnz_range(len, (uint64_t)low, (uint64_t)high, (uint64_t)rate);
    first.pop_back();  // the first row of every strip
    return first;
  };
  bool one_strip_only = true;
  for (uint64_t low : {512, 128, 32})
    for (uint64_t rate : {4, 8, 16})
      if (row_div_position_acc_to_exponential_increase_row_nnz_range({shortest_row, longest_row}, low, 2048, rate).size() > 2)
        one_strip_only = false;
  // Upstream's order is 1, 2, 3.  Where the vector is larger than an XCD's L2 cache and the longest row is far above
  // the average -- the matrices whose best graph is a coarse sort and two row strips -- strategy 3 goes first: its
  // winner is then known early (it is what a caller waits for), and it bounds what strategies 1 and 2 still sweep.
  // It leaves them a fifth of the budget.
  const bool sort_first = opt.only_dense_strategy == 0 && !one_strip_only &&
                          in.col_index_max + 1 > kL2BytesPerXcd / (in.val_dtype == DOUBLE ? 8 : 4) &&
                          longest_row >= 64 * std::max<uint64_t>(1, in.row.size() / row_len.size());
  // strategy 1: INPUT -> COMPRESS (a tenth of the budget, :5092)
  auto strategy1 = [&]() {
    if ((opt.only_dense_strategy == 0 || opt.only_dense_strategy == 1) && now_s() < T) {
      c.log("== dense strategy 1: INPUT -> COMPRESS" + c.stamp());
      if (sort_first) c.global = init_search_strategy(opt.struggle_step_num, T - now_s());
      BestGraph g;
      if (search_dense_strategy(c, in, {input, compress}, opt.only_dense_strategy == 1 || one_strip_only ? T : T / 10, g)) consider(g, "strategy1");
    }
  };
  // strategy 2: INPUT -> ROW_DIV by exponential row-length bands -> COMPRESS (a quarter of what is left, :5156)
  auto strategy2 = [&]() {
    if ((opt.only_dense_strategy == 0 || opt.only_dense_strategy == 2) && now_s() < T && !one_strip_only) {
      c.log("== dense strategy 2: INPUT -> DENSE_ROW_DIV -> COMPRESS" + c.stamp());
      c.global = init_search_strategy(opt.struggle_step_num, T - now_s());
      StrategyNode div = make_strategy(DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ_PARAM_STRATEGY, 32, 2048, 4, 0);
      const size_t strips = strips_of(row_len, 32, 2048, 4).size();
      const bool usable = strips >= 2 && strips <= 4;
      BestGraph g;
      if (usable && search_dense_strategy(c, in, {input, div, compress}, opt.only_dense_strategy == 2 ? T : (T - now_s()) / 4, g))
        consider(g, "strategy2");
      else if (!usable) c.log("strategy 2 skipped: row division yields 1 or more than 4 strips");
    }
  };
  // strategy 3: INPUT -> COARSE_SORT -> ROW_DIV(low x rate) -> COMPRESS (the rest, :4579-5039)
  auto strategy3 = [&]() {
    if ((opt.only_dense_strategy == 0 || opt.only_dense_strategy == 3) && now_s() < T && !one_strip_only) {
      c.log("== dense strategy 3: INPUT -> DENSE_ROW_COARSE_SORT -> DENSE_ROW_DIV -> COMPRESS" + c.stamp());
      StrategyNode sort = make_strategy(DENSE_ROW_COARSE_SORT_FIXED_PARAM_STRATEGY, 1);
      BestGraph best3;
      // (lowest, highest, rate) of the row-length bands.  First two strips only -- rows of at least
      // `lowest` elements and the rest -- which is what the LDS-tile kernel wants when x is larger
      // than an XCD's L2 cache; then the upstream grid 512/128/32 x 4/8/16 with bands up to 2048.
      std::vector<std::array<long, 3>> bands;
      if (in.col_index_max + 1 > kL2BytesPerXcd / (in.val_dtype == DOUBLE ? 8 : 4))
        for (long low : {48, 16, 256}) bands.push_back({low, low, 2});
      for (long low : {512, 128, 32})
        for (long rate : {4, 8, 16}) bands.push_back({low, 2048, rate});
      std::vector<std::vector<uint64_t>> seen;
      // A row division is a step of this level's search, and like the levels below it ends after steps in a row
      // that bring nothing (three here: a step costs seconds on a large matrix, not milliseconds).
      int struggle = 0;
      const double T3 = sort_first ? 0.8 * T : T;
    for (size_t bi = 0; bi < bands.size() && now_s() < T3; bi++) {
        StrategyNode div = make_strategy(DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ_PARAM_STRATEGY, bands[bi][0], bands[bi][1], bands[bi][2], 0);
        std::vector<uint64_t> cut = strips_of(sorted_len, bands[bi][0], bands[bi][1], bands[bi][2]);
        if (cut.size() > 4 || cut.size() < 2) continue;
        if (std::find(seen.begin(), seen.end(), cut) != seen.end()) continue;  // same strips as an earlier combination
        seen.push_back(cut);
        c.global = init_search_strategy(opt.struggle_step_num, T - now_s());
        BestGraph g;
        double budget = (T - now_s()) / 2;
        // another row division must lead by more than the noise of two timings (1 %), as launch settings must
        if (search_dense_strategy(c, in, {input, sort, div, compress}, budget, g) && g.gflops > best3.gflops * 1.01f) {
          best3 = g;
          struggle = 0;
        } else if (best3.gflops > 0 && ++struggle >= 3) {
          c.log("three row divisions in a row without an improvement: strategy 3 ends" + c.stamp());
          break;
        }
      }
      if (best3.gflops > 0) consider(best3, "strategy3");
    }
  };
  if (sort_first) {
    strategy3();
    strategy1();
    strategy2();
  } else {
    strategy1();
    strategy2();
    strategy3();
  }
  // strategies whose best graphs are within measurement noise of each other are measured again,
  // each over a region four times as long, and the faster one is kept
  {
    std::vector<BestGraph *> close;
    for (auto &g : finalists)
      if (g.gflops >= 0.93f * res.best.gflops) close.push_back(&g);
    if (close.size() >= 2) {
      SearchOptions longer = opt;
      longer.timed_region_ms = opt.timed_region_ms * 4;
      Ctx c2{longer, res, init_search_strategy(opt.struggle_step_num, 1e9), c.probe_x};
      float top = 0;
      for (BestGraph *g : close) {
        try {
          BuiltGraph bg = build_from_graph(in, *g, opt.wave);
          load_and_upload(*bg.builder, opt.device);
          if (as_hip_h2d(bg.builder->x.ptr, c.probe_x.data(), bg.builder->x.bytes) != 0) throw Error(as_hip_last_error());
          time_builder(c2, *bg.builder, g->time_ms, g->gflops);
          c.log("final comparison " + g->dense_strategy_name + ": " + std::to_string(g->gflops) + " GFLOP/s" + c.stamp());
          if (g->gflops > top) { top = g->gflops; res.best = *g; res.seconds_to_best = g->found_at_s; }
        } catch (const std::exception &e) {
          c.log(std::string("final comparison failed: ") + e.what());
        }
      }
    }
  }
  res.seconds = now_s();
  AS_CHECK(res.best.gflops > 0, "the search found no working candidate");
  res.log += convert_search_result_to_string(res.best.gflops, res.best.time_ms, res.best);
  return res;
}

}  // namespace asx
