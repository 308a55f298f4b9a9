// Operator graph: node kinds, node parameters, parameter strategies, and the
// executors that map each node onto one format operator (upstream
// exe_graph.hpp:36-202, parameter_set_strategy.hpp:7-22).
#pragma once
#include "matrix.hpp"
#include "op_manager.hpp"

namespace asx {

// Same order as upstream `enum exe_node_type` (exe_graph.hpp:36-57).
enum ExeNodeType : int {
  BEGIN_INPUT_FILE, BEGIN_ARTIFICIAL_INPUT, BEGIN_MEMORY_CACHE_INPUT_FILE, DENSE_ROW_COARSE_SORT, DENSE_FINE_SORT,
  DENSE_TOTAL_ROW_LEVEL_PADDING, DENSE_BLOCK_SORT, DENSE_ROW_DIV, DENSE_FIXED_COL_DIV, COMPRESS,
  COMPRESSED_ROW_PADDING, COMPRESSED_BLOCK_SORT, COMPRESSED_THREAD_LEVEL_ROW_DIV, COMPRESSED_THREAD_LEVEL_COL_DIV,
  COMPRESSED_WARP_LEVEL_ROW_DIV, COMPRESSED_WARP_LEVEL_COL_DIV, COMPRESSED_TBLOCK_LEVEL_ROW_DIV,
  COMPRESSED_TBLOCK_LEVEL_COL_DIV, COMPRESSED_THREAD_LEVEL_NNZ_DIV, EXE_NODE_TYPE_COUNT
};
const char *convert_exe_node_type_to_string(ExeNodeType t);  // exe_graph.cc:2574

// Concrete node parameters: one struct carrying the fields of every upstream
// exe_*_param_t (exe_graph.hpp:60-150); a node kind reads only its own fields.
struct ExeNode {
  ExeNodeType type = COMPRESS;
  long multiply = 0, padding_row_length = 0;                 // COMPRESSED_ROW_PADDING
  long TLB_nnz_num = 0;                                      // COMPRESSED_THREAD_LEVEL_NNZ_DIV
  std::vector<uint64_t> col_num_of_TLB_in_each_parent_block; // COMPRESSED_THREAD_LEVEL_COL_DIV
  std::vector<uint32_t> row_num_of_each_BLB;                 // COMPRESSED_TBLOCK_LEVEL_ROW_DIV
  // COMPRESSED_WARP_LEVEL_ROW_DIV / _COL_DIV, COMPRESSED_TBLOCK_LEVEL_COL_DIV
  std::vector<std::vector<uint32_t>> nested_block_size;
  std::vector<uint64_t> bin_row_nnz_low_bound;               // DENSE_ROW_COARSE_SORT
  std::vector<uint64_t> first_row_of_each_sort_band;         // DENSE_FINE_SORT (empty: one band)
  std::vector<uint64_t> sort_block_index_arr;                // COMPRESSED_BLOCK_SORT (empty: every BLB)
  std::vector<uint64_t> row_div_position;                    // DENSE_ROW_DIV
  // DENSE_ROW_DIV, DENSE_FIXED_COL_DIV: the sub-block of an already divided matrix that is cut (exe_graph.hpp
  // exe_dense_row_div_param_t / exe_dense_fixed_col_div_param_t); 0 for the first division of the matrix
  uint64_t dense_sub_block_id = 0;
  long fixed_col_block_size = 0;                             // DENSE_FIXED_COL_DIV
  // DENSE_ROW_DIV of a sub-block into strips of equal height (upstream fixed_len_row_div, op_manager.cc:127, an
  // operator without a node of its own): used when row_div_position is empty
  long fixed_row_block_size = 0;
  // COMPRESSED_TBLOCK_LEVEL_COL_DIV into 2-D tiles (row_group != 0): slice width, group height, BLB size
  uint64_t col_slice = 0, row_group = 0, block_nnz = 0;
  void reset_param();
};

// execute_exe_*_node (exe_graph.cc:1443-2340).  Dense nodes act on the whole
// matrix; compressed nodes on one sub-matrix and insert the default BLB / WLB
// levels they depend on, exactly as upstream does.
void execute_dense_node(Matrix &m, const ExeNode &node);
void execute_exe_node_in_compressed_sub_matrix(Matrix &m, uint64_t sub, const ExeNode &node);  // exe_graph.cc:2795
// execute_default_div_to_complete_each_level_blocking (default_auto_tuner.cc:384-447)
void execute_default_div_to_complete_each_level_blocking(Matrix &m, uint64_t sub);

// Same order as upstream `enum exe_node_param_set_strategy`.
enum ParamStrategy : int {
  COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY,
  COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY,
  COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY,
  COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY,
  COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY,
  COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY,
  COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY,
  COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY,
  COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT_PARAM_STRATEGY,
  DENSE_ROW_COARSE_SORT_FIXED_PARAM_STRATEGY,
  DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY,
  COMPRESS_NONE_PARAM_STRATEGY,
  DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ_PARAM_STRATEGY,
  // No upstream counterpart: cuts every row where its columns cross a multiple of p0 (the column
  // slice an LDS-resident part of x covers), so each BLB reads x from one slice only.
  COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE_PARAM_STRATEGY,
  // No upstream counterpart: 2-D tiles of p1 rows x p0 columns, elements re-ordered tile by tile,
  // every tile cut into BLBs of at most p2 elements (x slice and the row group's sums live in LDS).
  COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY,
  PARAM_STRATEGY_COUNT
};
const char *convert_param_set_strategy_to_string(ParamStrategy s);
ExeNodeType node_type_of_strategy(ParamStrategy s);

// param_strategy_node_t: a scalar-knob strategy plus the node it parameterises.
// Knob meaning per strategy (parameter_set_strategy.hpp:24-110):
//   ROW_PADDING_DIRECT        p0 = multiply, p1 = padding_row_length
//   BLB_ROW_DIV_EVENLY        p0 = block_row_num
//   BLB_ROW_DIV_LEAST_NNZ     p0 = nnz_low_bound
//   BLB/WLB/TLB_COL_DIV_FIXED p0 = col_block_nnz_num
//   WLB_ROW_DIV_EVENLY        p0 = warp_row_num_of_each_BLB
//   TLB_NNZ_DIV_DIRECT        p0 = block_nnz_num
//   COARSE_SORT_FIXED         p0 = row_nnz_low_bound_step_size
//   BLB_COL_DIV_COL_SLICE     p0 = col_slice_width
//   BLB_COL_DIV_ROW_GROUP_COL_SLICE  p0 = col_slice_width, p1 = row_group_size, p2 = block_nnz_num
//   DENSE_ROW_DIV_EXP         p0 = lowest, p1 = highest, p2 = expansion_rate, p3 = sub_dense_block_id
struct StrategyNode {
  ParamStrategy strategy = COMPRESS_NONE_PARAM_STRATEGY;
  long p[4] = {0, 0, 0, 0};
  ExeNode node;
  // only for DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE (report needs nnz / dtype / max indices)
  uint64_t in_nnz = 0, in_col_index_max = 0, in_row_index_max = 0;
  DType in_val_dtype = FLOAT;
};
StrategyNode make_strategy(ParamStrategy s, long p0 = 0, long p1 = 0, long p2 = 0, long p3 = 0);

// execute_param_strategy_node_of_dense_matrix / _of_sub_compressed_matrix
// (parameter_set_strategy.cc:193-592): fill node params from the matrix.
void execute_param_strategy_node_of_dense_matrix(StrategyNode &n, Matrix &m);
void execute_param_strategy_node_of_sub_compressed_matrix(StrategyNode &n, Matrix &m, uint64_t sub);

// Report text (parameter_set_strategy.cc:1119-1345).
std::string convert_strategy_param_to_string(const StrategyNode &n);
std::string convert_stategy_node_to_string(const StrategyNode &n);
std::string convert_all_stategy_node_of_sub_matrix_to_string(const std::vector<StrategyNode> &v);

}  // namespace asx
