// Search engine: which operator graphs, parameters and templates are tried, in which order, and when
// to stop.  Follows the upstream white-list search (whilte_list_path_impl.cc, default_auto_tuner.cc,
// search_strategy.cc, param_enumerater.cc, matrix_info.cc) with every candidate evaluated in-process
// (hipRTC + launches timed with events) and the enumeration ranges set for 64-lane wavefronts,
// 1024-thread workgroups, 64 KB LDS per workgroup and 256 CUs.
#pragma once
#include <chrono>
#include <functional>

#include "code_builder.hpp"
#include "exe_graph.hpp"

namespace asx {

// matrix_info_t (matrix_info.hpp:7-17)
struct MatrixInfo {
  std::vector<uint64_t> row_nnz;
  uint64_t nnz = 0, row_num = 0, col_num = 0, max_row_nnz = 0, min_row_nnz = 0, avg_row_nnz = 0;
  bool is_sorted = false;
  bool is_double = false;   // value type of the matrix
  // 4, 3 or 2 where the first rows come in blocks of that many consecutive rows with the same columns (the dense
  // blocks of a FEM matrix), else 1; only get_sub_matrix_info_from_compressed_matrix_block fills it
  uint64_t row_block = 1;
  // distinct diagonals (column - row) the elements lie on, counted up to 65 (65 = more); 0 = not counted (rows of
  // more than 64 elements); only get_sub_matrix_info_from_compressed_matrix_block fills it.  A stencil has as many
  // as its longest row has elements: the ELL template then needs no column array at all.
  uint64_t diagonals = 0;
};
MatrixInfo get_matrix_info(const Matrix &m);                                      // matrix_info.cc:22
MatrixInfo get_sub_matrix_info_from_compressed_matrix_block(const Matrix &m, uint64_t sub);  // matrix_info.cc:140

// param_enumerater_t (param_enumerater.hpp): odometer over integer knobs, knob 0 fastest,
// optional filters that veto a combination.
struct ParamEnumerator {
  struct Knob { long *ptr; long low, up, step; };
  std::vector<Knob> knobs;
  std::vector<std::function<bool()>> filters;
  bool started = false;
  void add(long *ptr, long low, long up, long step);     // register_integer_independ_param_to_enumerater
  void add_filter(std::function<bool()> f) { filters.push_back(std::move(f)); }
  // set_param_combination_to_next: advance to the next accepted combination; false when exhausted
  bool next();
};

// search_strategy_t (search_strategy.hpp:7-14) and continue_search (search_strategy.cc:24-102)
struct SearchStrategy {
  uint64_t remain_step_num = 10, struggle_step_num = 10;
  std::chrono::steady_clock::time_point begin_time;
  double total_allow_search_time = 0;
  float best_glops = 0;
};
SearchStrategy init_search_strategy(uint64_t struggle_step_num, double total_allow_search_time);
bool continue_search(SearchStrategy &s, float gflops);
bool continue_search(const SearchStrategy &s);

// template_node_t + per-template launch parameters (exe_graph.hpp:405-475)
struct TemplateNode {
  TemplateType type = NONE_TEMPLATE;
  long tblock_num = 0, thread_num_in_block = 0, thread_num_of_row_reduce = 1, vec_width = 1;
  // 1: columns stored as 16-bit differences to the unit number (set_relative_columns); 2: computed from the
  // slot's diagonal, no column array (set_diagonal_columns); 3: tile template in its column-run form
  // (set_column_runs)
  long col_relative = 0;
  // 1: tile template under row ownership (set_row_ownership)
  long own_rows = 0;
  long row_block = 0;   // tile template: rows stored in blocks of this many (as_builder_set_row_blocks), 0 = not
};
std::string convert_template_node_to_string(const TemplateNode &n);   // exe_graph.cc:3317

// compressed_sub_block_exe_graph_and_template_t
struct SubGraph {
  std::vector<StrategyNode> nodes;
  TemplateNode tpl;
  float gflops = 0, time_ms = 0;
  uint64_t format_bytes = 0;  // bytes the kernel moves per launch: format arrays, x once, the strip's rows of y once
  double found_at_s = 0;  // seconds into the search at which this candidate was measured
};
// dense_view_matrix_and_compressed_sub_block_exe_graph_and_template_t
struct BestGraph {
  std::vector<StrategyNode> dense;   // INPUT [, COARSE_SORT] [, ROW_DIV], COMPRESS
  std::vector<SubGraph> subs;
  float gflops = 0, time_ms = 0;
  std::string dense_strategy_name;   // "strategy1" | "strategy2" | "strategy3"
  // the kernels of the strips run one after the other instead of on concurrent streams (measured faster)
  bool serial_launch = false;
  // rows without elements were removed from the input before the first operator
  bool empty_rows_removed = false;
  // seconds into the search at which this graph was measured as a whole
  double found_at_s = 0;
};
// convert_dense_view_matrix_and_compressed_sub_block_exe_graph_and_template_to_string_safety
// (whilte_list_path_impl.cc:4150)
std::string convert_graph_to_string(const BestGraph &g);
// the lines upstream's main prints around it (main.cc:646-657), up to and including "finish search"
std::string convert_search_result_to_string(float gflops, float time_ms, const BestGraph &g);

struct SearchOptions {
  double total_time_s = 120;        // upstream: 32400
  uint64_t struggle_step_num = 10;  // upstream main.cc:634
  double padding_rate_up_bound = 4; // global_config.json PADDING_RATE_UP_BOUND
  int device = 0;
  unsigned wave = 64;
  double timed_region_ms = 20;      // per candidate, after warm-up
  std::string checkpoint_dir;       // best_result_of_strategy{1,2,3} written here when not empty
  bool verbose = false;
  int only_dense_strategy = 0;      // 0 = all, 1/2/3 = just that one
  // false: an input with rows that hold no element is rejected, as upstream does (main.cc:604-621);
  // true: such rows are removed before the first operator of every graph (remove_empty_rows)
  bool remove_empty_rows = false;
  // true: the two general templates DIRECT_ATOM / SHARED_MEMORY, which upstream implements
  // (direct_atom_op.cc, shared_memory_op.cc) but keeps out of its white list, are searched as well
  bool general_templates = false;
  // every candidate's y for x[j] = 1 + j % 7 is compared with a host CSR product (computed once per search) before it is timed; a candidate
  // that differs counts as failed and cannot win
  bool verify_candidates = true;
};

struct SearchResult {
  BestGraph best;
  uint64_t candidates = 0, failed_candidates = 0;
  double seconds = 0, seconds_to_best = 0;
  std::string log;   // what upstream prints to test.log: per-candidate lines + the final report
};

// find_best_graph_of_white_list_strategy (whilte_list_path_impl.cc:5041)
SearchResult find_best_graph_of_white_list_strategy(const CooInput &in, const SearchOptions &opt);

// execute_dense_view_matrix_and_compressed_sub_block_exe_graph_and_template (:5318): rebuild the
// format from a graph and return a builder with every template set, compressed and launch-configured.
struct BuiltGraph {
  std::unique_ptr<Matrix> matrix;
  std::unique_ptr<Builder> builder;
};
BuiltGraph build_from_graph(const CooInput &in, const BestGraph &g, unsigned wave);

}  // namespace asx
