#include "exe_graph.hpp"

#include "graph_enumerate.hpp"

namespace asx {

const char *convert_exe_node_type_to_string(ExeNodeType t) {
  static const char *n[] = {"BEGIN_INPUT_FILE", "BEGIN_ARTIFICIAL_INPUT", "BEGIN_MEMORY_CACHE_INPUT_FILE",
                            "DENSE_ROW_COARSE_SORT", "DENSE_FINE_SORT", "DENSE_TOTAL_ROW_LEVEL_PADDING",
                            "DENSE_BLOCK_SORT", "DENSE_ROW_DIV", "DENSE_FIXED_COL_DIV", "COMPRESS",
                            "COMPRESSED_ROW_PADDING", "COMPRESSED_BLOCK_SORT", "COMPRESSED_THREAD_LEVEL_ROW_DIV",
                            "COMPRESSED_THREAD_LEVEL_COL_DIV", "COMPRESSED_WARP_LEVEL_ROW_DIV",
                            "COMPRESSED_WARP_LEVEL_COL_DIV", "COMPRESSED_TBLOCK_LEVEL_ROW_DIV",
                            "COMPRESSED_TBLOCK_LEVEL_COL_DIV", "COMPRESSED_THREAD_LEVEL_NNZ_DIV"};
  AS_CHECK(t >= 0 && t < EXE_NODE_TYPE_COUNT, "unknown node type");
  return n[(int)t];
}

void ExeNode::reset_param() {
  ExeNodeType t = type;
  *this = ExeNode();
  type = t;
}

// execute_exe_dense_row_div_node (exe_graph.cc:1574), _coarse_sort_node (:1642),
// _compress_node (:1518)
void execute_dense_node(Matrix &m, const ExeNode &node) {
  switch (node.type) {
    case BEGIN_MEMORY_CACHE_INPUT_FILE:
    case BEGIN_INPUT_FILE:
      return;  // the matrix already exists when a node is executed on it
    case DENSE_ROW_COARSE_SORT:
      total_dense_block_coarse_sort(m, node.bin_row_nnz_low_bound);
      return;
    case DENSE_FINE_SORT:  // op_manager API upstream (no node executor there)
      total_dense_block_sort(m, node.first_row_of_each_sort_band);
      return;
    case DENSE_ROW_DIV:  // exe_graph.cc:1574-1613: the whole matrix first, a sub-block of the table afterwards
      if (m.items.empty()) {
        AS_CHECK(node.dense_sub_block_id == 0, "the matrix has no sub-blocks yet");
        if (node.row_div_position.size() <= 2) return;  // a single strip is a no-op
        var_len_row_div(m, node.row_div_position);
      } else if (node.row_div_position.empty() && node.fixed_row_block_size > 0) {
        fixed_len_row_div(m, (uint64_t)node.fixed_row_block_size, node.dense_sub_block_id);
      } else {
        var_len_row_div(m, node.row_div_position, node.dense_sub_block_id);
      }
      return;
    case DENSE_FIXED_COL_DIV:  // exe_graph.cc:1615-1640
      AS_CHECK(node.fixed_col_block_size > 0, "band width must be positive");
      if (m.items.empty()) {
        AS_CHECK(node.dense_sub_block_id == 0, "the matrix has no sub-blocks yet");
        fixed_len_col_div(m, (uint64_t)node.fixed_col_block_size);
      } else {
        fixed_len_col_div(m, (uint64_t)node.fixed_col_block_size, node.dense_sub_block_id);
      }
      return;
    case COMPRESS:
      compress_dense_view(m);
      return;
    default:
      throw Error(std::string("execute_dense_node: node type is not supported in the dense sub-graph: ") +
                  convert_exe_node_type_to_string(node.type));
  }
}

static void need_levels(CompressedBlock &cb, size_t want) {
  if (want >= 3 && cb.read_index.size() == 2) default_sep_tblock_level_row_csr(cb);
  if (want >= 4 && cb.read_index.size() == 3) default_sep_warp_level_row_csr(cb);
}

static std::vector<uint64_t> iota_ids(size_t n) {
  std::vector<uint64_t> v(n);
  for (size_t i = 0; i < n; i++) v[i] = i;
  return v;
}

void execute_exe_node_in_compressed_sub_matrix(Matrix &m, uint64_t sub, const ExeNode &node) {
  CompressedBlock &cb = m.block(sub);
  switch (node.type) {
    case COMPRESSED_ROW_PADDING:  // exe_graph.cc:2311
      AS_CHECK(cb.read_index.size() == 2, "row padding must come first");
      compress_block_end_block_multiple_padding(m, sub, node.multiply, node.padding_row_length);
      return;
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV:  // exe_graph.cc:1688
      AS_CHECK(cb.read_index.size() == 2, "BLB level already exists");
      sep_tblock_level_row_csr(cb, node.row_num_of_each_BLB);
      return;
    case COMPRESSED_BLOCK_SORT: {  // op_manager API upstream (no node executor there)
      AS_CHECK(!m.sorted_row_index.present, "a sort inside BLBs excludes a sort of the whole matrix (and remove_empty_rows)");
      AS_CHECK(cb.read_index.size() == 3, "the BLB level must exist and be the last one");
      compressed_block_sort(cb, node.sort_block_index_arr.empty() ? iota_ids(cb.read_index[2]->block_num) : node.sort_block_index_arr,
                            m.items[sub].max_row - m.items[sub].min_row + 1);
      return;
    }
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV: {  // exe_graph.cc:1754
      AS_CHECK(cb.read_index.size() == 2, "BLB level already exists");
      if (node.row_group != 0) {  // 2-D tiles (no upstream counterpart)
        sep_tblock_level_row_group_col_slice(cb, node.col_slice, node.row_group, node.block_nnz);
        return;
      }
      one_row_sep_tblock_level_row_csr(cb);
      AS_CHECK(cb.read_index[2]->block_num == node.nested_block_size.size(), "one size list per non-empty row");
      sep_tblock_level_col_csr(cb, iota_ids(node.nested_block_size.size()), node.nested_block_size);
      return;
    }
    case COMPRESSED_WARP_LEVEL_ROW_DIV: {  // exe_graph.cc:1841
      AS_CHECK(cb.read_index.size() == 2 || cb.read_index.size() == 3, "WLB level already exists");
      need_levels(cb, 3);
      AS_CHECK(cb.read_index[2]->block_num == node.nested_block_size.size(), "one size list per BLB");
      sep_warp_level_row_csr(cb, iota_ids(node.nested_block_size.size()), node.nested_block_size);
      return;
    }
    case COMPRESSED_WARP_LEVEL_COL_DIV: {  // exe_graph.cc:1942
      AS_CHECK(cb.read_index.size() == 2 || cb.read_index.size() == 3, "WLB level already exists");
      need_levels(cb, 3);
      one_row_sep_warp_level_row_csr(cb);
      AS_CHECK(cb.read_index[3]->block_num == node.nested_block_size.size(), "one size list per non-empty row");
      sep_warp_level_col_csr(cb, iota_ids(node.nested_block_size.size()), node.nested_block_size);
      return;
    }
    case COMPRESSED_THREAD_LEVEL_ROW_DIV:  // exe_graph.cc:2043
      AS_CHECK(cb.read_index.size() >= 2 && cb.read_index.size() <= 4, "TLB level already exists");
      need_levels(cb, 4);
      sep_thread_level_col_ell_with_padding(cb, {}, {}, m.wave);
      return;
    case COMPRESSED_THREAD_LEVEL_COL_DIV:  // exe_graph.cc:2152
      AS_CHECK(cb.read_index.size() >= 2 && cb.read_index.size() <= 4, "TLB level already exists");
      need_levels(cb, 4);
      AS_CHECK(node.col_num_of_TLB_in_each_parent_block.size() == cb.read_index[3]->block_num, "one TLB size per WLB");
      sep_thread_level_col_ell_with_padding(cb, iota_ids(node.col_num_of_TLB_in_each_parent_block.size()),
                                            node.col_num_of_TLB_in_each_parent_block, m.wave);
      return;
    case COMPRESSED_THREAD_LEVEL_NNZ_DIV:  // exe_graph.cc:2248
      AS_CHECK(cb.read_index.size() == 2, "nnz division needs an undivided sub-matrix");
      need_levels(cb, 4);
      sep_thread_level_acc_to_nnz(cb, (uint64_t)node.TLB_nnz_num);
      return;
    default:
      throw Error(std::string("execute_exe_node_in_compressed_sub_matrix: node type is not supported: ") +
                  convert_exe_node_type_to_string(node.type));
  }
}

// Missing levels: 1 BLB = whole sub-matrix, 1 WLB per BLB, TLB size 1 everywhere.
void execute_default_div_to_complete_each_level_blocking(Matrix &m, uint64_t sub) {
  CompressedBlock &cb = m.block(sub);
  need_levels(cb, 4);
  if (cb.read_index.size() == 4) {
    uint64_t n = cb.read_index[3]->block_num;
    sep_thread_level_col_ell_with_padding(cb, iota_ids(n), std::vector<uint64_t>(n, 1), m.wave);
  }
  AS_CHECK(cb.read_index.size() == 7, "blocking is incomplete");
}

// ---------------------------------------------------------------------------
static const struct { const char *name; ExeNodeType node; } kStrategy[] = {
    {"COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY", COMPRESSED_ROW_PADDING},
    {"COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY", COMPRESSED_TBLOCK_LEVEL_ROW_DIV},
    {"COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY", COMPRESSED_TBLOCK_LEVEL_ROW_DIV},
    {"COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY", COMPRESSED_TBLOCK_LEVEL_COL_DIV},
    {"COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY", COMPRESSED_WARP_LEVEL_ROW_DIV},
    {"COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY", COMPRESSED_WARP_LEVEL_COL_DIV},
    {"COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY", COMPRESSED_THREAD_LEVEL_ROW_DIV},
    {"COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY", COMPRESSED_THREAD_LEVEL_COL_DIV},
    {"COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT_PARAM_STRATEGY", COMPRESSED_THREAD_LEVEL_NNZ_DIV},
    {"DENSE_ROW_COARSE_SORT_FIXED_PARAM_STRATEGY", DENSE_ROW_COARSE_SORT},
    {"DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY", BEGIN_MEMORY_CACHE_INPUT_FILE},
    {"COMPRESS_NONE_PARAM_STRATEGY", COMPRESS},
    {"DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ_PARAM_STRATEGY", DENSE_ROW_DIV},
    {"COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE_PARAM_STRATEGY", COMPRESSED_TBLOCK_LEVEL_COL_DIV},
    {"COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY", COMPRESSED_TBLOCK_LEVEL_COL_DIV},
};

const char *convert_param_set_strategy_to_string(ParamStrategy s) {
  AS_CHECK(s >= 0 && s < PARAM_STRATEGY_COUNT, "strategy type is not supported");
  return kStrategy[(int)s].name;
}
ExeNodeType node_type_of_strategy(ParamStrategy s) {
  AS_CHECK(s >= 0 && s < PARAM_STRATEGY_COUNT, "strategy type is not supported");
  return kStrategy[(int)s].node;
}

StrategyNode make_strategy(ParamStrategy s, long p0, long p1, long p2, long p3) {
  StrategyNode n;
  n.strategy = s;
  n.p[0] = p0; n.p[1] = p1; n.p[2] = p2; n.p[3] = p3;
  n.node.type = node_type_of_strategy(s);
  return n;
}

void execute_param_strategy_node_of_dense_matrix(StrategyNode &n, Matrix &m) {
  n.node.reset_param();
  switch (n.strategy) {
    case DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY:
    case COMPRESS_NONE_PARAM_STRATEGY:
      return;
    case DENSE_ROW_COARSE_SORT_FIXED_PARAM_STRATEGY: {  // parameter_set_strategy.cc:441-501
      AS_CHECK(!m.is_sorted && !m.is_blocked && !m.is_compressed, "coarse sort must be the first dense operator");
      AS_CHECK(n.p[0] > 0, "step size must be positive");
      std::vector<uint64_t> len = get_nnz_of_each_row(m);
      if (n.p[0] == 1) {
        n.node.bin_row_nnz_low_bound = bin_row_nnz_low_bound_of_fixed_granularity_coar_sort(len, 1);
      } else {
        uint64_t mn = len[0], mx = len[0];
        for (uint64_t l : len) { mn = std::min(mn, l); mx = std::max(mx, l); }
        for (uint64_t i = mn; i <= mx; i += (uint64_t)n.p[0]) n.node.bin_row_nnz_low_bound.push_back(i == mn ? 0 : i);
      }
      return;
    }
    case DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ_PARAM_STRATEGY: {  // :534-592
      AS_CHECK(n.p[2] > 0 && n.p[0] > 0, "expansion rate and lowest bound must be positive");
      n.node.dense_sub_block_id = (uint64_t)n.p[3];
      if (m.items.empty()) {
        AS_CHECK(n.p[3] == 0, "the matrix has no sub-blocks yet");
        n.node.row_div_position = row_div_position_acc_to_exponential_increase_row_nnz_range(
            get_nnz_of_each_row(m), (uint64_t)n.p[0], (uint64_t)n.p[1], (uint64_t)n.p[2]);
      } else {
        // the bands of row length inside one sub-block (rows relative to its first row)
        AS_CHECK((uint64_t)n.p[3] < m.items.size(), "sub-matrix id out of range");
        const DenseItem &it = m.items[(size_t)n.p[3]];
        std::vector<uint64_t> len(it.max_row - it.min_row + 1, 0);
        for (uint64_t k = it.begin_coo; k <= it.end_coo; k++) len[m.coo_row[k] - it.min_row]++;
        n.node.row_div_position = row_div_position_acc_to_exponential_increase_row_nnz_range(len, (uint64_t)n.p[0], (uint64_t)n.p[1], (uint64_t)n.p[2]);
      }
      return;
    }
    default:
      throw Error("execute_param_strategy_node_of_dense_matrix: not a dense-view strategy");
  }
}

void execute_param_strategy_node_of_sub_compressed_matrix(StrategyNode &n, Matrix &m, uint64_t sub) {
  CompressedBlock &cb = m.block(sub);
  n.node.reset_param();
  auto sub_rows = [&]() { return cb.read_index[0]->max_row - cb.read_index[0]->min_row + 1; };
  switch (n.strategy) {
    case COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY:
      AS_CHECK(cb.read_index.size() == 2 && n.p[0] > 0 && n.p[1] > 0, "bad row padding parameters");
      n.node.multiply = n.p[0];
      n.node.padding_row_length = n.p[1];
      return;
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY:
      AS_CHECK(cb.read_index.size() == 2 && n.p[0] > 0, "bad BLB row division parameters");
      for (uint64_t s : row_block_size_of_a_sub_matrix_by_fixed_div(sub_rows(), (uint64_t)n.p[0]))
        n.node.row_num_of_each_BLB.push_back((uint32_t)s);
      return;
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY:
      AS_CHECK(cb.read_index.size() == 2 && n.p[0] > 0, "bad BLB row division parameters");
      for (uint64_t s : row_block_size_of_a_sub_matrix_by_nnz_low_bound(get_nnz_of_each_row_in_compressed_sub_matrix(cb),
                                                                        (uint64_t)n.p[0]))
        n.node.row_num_of_each_BLB.push_back((uint32_t)s);
      return;
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY:
      AS_CHECK(cb.read_index.size() == 2 && n.p[0] > 0, "bad BLB column division parameters");
      n.node.nested_block_size = col_block_size_of_each_row(get_nnz_of_each_row_in_compressed_sub_matrix(cb), (uint64_t)n.p[0]);
      return;
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE_PARAM_STRATEGY: {
      AS_CHECK(cb.read_index.size() == 2 && n.p[0] > 0, "bad column slice width");
      const Index &ri = *cb.read_index[0], &ci = *cb.read_index[1];
      n.node.nested_block_size = col_block_size_of_each_row_by_col_slice(ri.index_arr.v, ci.index_arr.v, (uint64_t)n.p[0]);
      cb.col_slice = (uint64_t)n.p[0];
      return;
    }
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY:
      AS_CHECK(cb.read_index.size() == 2 && n.p[0] > 0 && n.p[1] > 0 && n.p[2] > 0, "bad tile division parameters");
      n.node.col_slice = (uint64_t)n.p[0];
      n.node.row_group = (uint64_t)n.p[1];
      n.node.block_nnz = (uint64_t)n.p[2];
      return;
    case COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY: {
      AS_CHECK(cb.read_index.size() <= 3 && n.p[0] > 0, "bad WLB row division parameters");
      need_levels(cb, 3);
      n.node.nested_block_size = row_block_size_of_each_sub_block_by_fixed_div(cb.read_index[2]->row_number.v, (uint64_t)n.p[0]);
      return;
    }
    case COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: {
      AS_CHECK(cb.read_index.size() <= 3 && n.p[0] > 0, "bad WLB column division parameters");
      need_levels(cb, 3);
      const IArr &fr = cb.read_index[2]->first_row;
      for (size_t i = 0; i + 1 < fr.size(); i++) AS_CHECK(fr[i] < fr[i + 1], "BLBs must not share rows");
      n.node.nested_block_size =
          col_block_size_of_each_row_without_block_merge(get_nnz_of_each_row_in_compressed_sub_matrix(cb), (uint64_t)n.p[0]);
      return;
    }
    case COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY:
      AS_CHECK(cb.read_index.size() <= 4, "TLB level already exists");
      return;
    case COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY:
      AS_CHECK(cb.read_index.size() <= 4 && n.p[0] > 0, "bad TLB column division parameters");
      need_levels(cb, 4);
      n.node.col_num_of_TLB_in_each_parent_block = col_div_of_TLB_global_fixed_col_size(cb.read_index[3]->block_num, (uint64_t)n.p[0]);
      return;
    case COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT_PARAM_STRATEGY:
      AS_CHECK(cb.read_index.size() == 2 && n.p[0] > 0, "bad nnz division parameters");
      n.node.TLB_nnz_num = n.p[0];
      return;
    default:
      throw Error("execute_param_strategy_node_of_sub_compressed_matrix: not a compressed-view strategy");
  }
}

std::string convert_strategy_param_to_string(const StrategyNode &n) {
  auto kv = [](const char *k, long v) { return std::string(k) + ":" + std::to_string(v) + "\n"; };
  std::string s;
  switch (n.strategy) {
    case COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY:
      return "{\n" + kv("multiply", n.p[0]) + kv("padding_row_length", n.p[1]) + "}\n";
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY:
      return "{\n" + kv("block_row_num", n.p[0]) + "}\n";
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY:
      return "{\n" + kv("nnz_low_bound", n.p[0]) + "}\n";
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY:
    case COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY:
    case COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY:
      return "{\n" + kv("col_block_nnz_num", n.p[0]) + "}\n";
    case COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY:
      return "{\n" + kv("warp_row_num_of_each_BLB", n.p[0]) + "}\n";
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE_PARAM_STRATEGY:
      return "{\n" + kv("col_slice_width", n.p[0]) + "}\n";
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY:
      return "{\n" + kv("col_slice_width", n.p[0]) + kv("row_group_size", n.p[1]) + kv("block_nnz_num", n.p[2]) + "}\n";
    case COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY:
      return "{\n}\n";
    case COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT_PARAM_STRATEGY:
      return "{\n" + kv("block_nnz_num", n.p[0]) + "}\n";
    case DENSE_ROW_COARSE_SORT_FIXED_PARAM_STRATEGY:
      return "{\n" + kv("row_nnz_low_bound_step_size", n.p[0]) + "}\n";
    case DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY:
      return "{\n" + kv("nnz", (long)n.in_nnz) + "data_type:" + dtype_name(n.in_val_dtype) + "\n" +
             kv("col_index_max", (long)n.in_col_index_max) + kv("row_index_max", (long)n.in_row_index_max) + "}\n";
    case COMPRESS_NONE_PARAM_STRATEGY:
      return "";
    case DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ_PARAM_STRATEGY:
      return "{\n" + kv("expansion_rate", n.p[2]) + kv("lowest_nnz_bound_of_row", n.p[0]) +
             kv("highest_nnz_bound_of_row", n.p[1]) + kv("sub_dense_block_id", n.p[3]) + "}\n";
    default:
      throw Error("convert_strategy_param_to_string: strategy type is not supported");
  }
}

std::string convert_stategy_node_to_string(const StrategyNode &n) {
  return std::string("{\n") + "strategy_type:" + convert_param_set_strategy_to_string(n.strategy) + "\n" +
         "node_type:" + convert_exe_node_type_to_string(n.node.type) + "\n" + convert_strategy_param_to_string(n) + "}\n";
}

std::string convert_all_stategy_node_of_sub_matrix_to_string(const std::vector<StrategyNode> &v) {
  std::string s;
  for (auto &n : v) s += convert_stategy_node_to_string(n);
  return s;
}

}  // namespace asx
