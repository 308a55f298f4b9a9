// Dump harness around the UPSTREAM host code (test infrastructure only).
//
// Compiled together with the upstream object files into oracle/_ref/libasref.so
// (see Makefile, target `ref`).  It drives the upstream operators through the
// upstream node executors and exposes the resulting arrays with the same
// (sub, slot, field) addressing as as_matrix_get_u64 / as_matrix_get_f64 of the
// product library, so tests can compare the two element by element.
//
// Upstream aborts the process on invalid input (live asserts); callers must
// only pass operator sequences that are valid upstream.
#include <unistd.h>

#include <cstring>
#include <iostream>
#include <sstream>
#include <vector>

#include "exe_graph.hpp"
#include "parameter_set_strategy.hpp"
#include "default_auto_tuner.hpp"
#include "param_enumerater.hpp"
#include "search_strategy.hpp"

namespace {
struct Quiet {  // upstream logs to std::cout on every call
  std::streambuf *old;
  Quiet() : old(std::cout.rdbuf(nullptr)) {}
  ~Quiet() { std::cout.rdbuf(old); }
};
struct RefMatrix {
  sparse_struct_t *m = nullptr;
  operator_manager_t *op = nullptr;
  code_builder_t *builder = nullptr;
  std::vector<void *> templates;           // per sub-matrix
  std::vector<template_type> template_types;
};
int64_t put(const void *arr, data_type dt, uint64_t n, uint64_t *out, uint64_t cap, int *dtype) {
  if (arr == NULL) return -1;
  if (dtype) *dtype = (int)dt;
  if (out)
    for (uint64_t i = 0; i < n && i < cap; i++) out[i] = read_from_array_with_data_type((void *)arr, dt, i);
  return (int64_t)n;
}
}  // namespace

extern "C" {

// chdir to the directory holding the redirected global_config.json
int ref_init(const char *config_dir) { return chdir(config_dir); }

// The reference's own reader of .mtx.coo text (struct.cc:92-175).  Returns the number of entries; copies
// min(nnz, cap) of them (0-based indices, values widened to double) and header = {max row index, max column index}.
int64_t ref_read_coo_file(const char *path, int val_dtype, uint64_t *row, uint64_t *col, double *val, uint64_t cap,
                          uint64_t header[2]) {
  Quiet q;
  vector<unsigned long> r, c;
  vector<float> vf;
  vector<double> vd;
  unsigned long max_row = 0, max_col = 0;
  get_matrix_index_and_val_from_file(path, r, c, vf, vd, (data_type)val_dtype, max_row, max_col);
  for (uint64_t i = 0; i < r.size() && i < cap; i++) {
    row[i] = r[i];
    col[i] = c[i];
    val[i] = val_dtype == FLOAT ? (double)vf[i] : vd[i];
  }
  if (header) { header[0] = max_row; header[1] = max_col; }
  return (int64_t)r.size();
}

void *ref_matrix_from_coo(uint64_t rows, uint64_t cols, uint64_t nnz, const uint64_t *row, const uint64_t *col,
                          const double *val, int val_dtype) {
  Quiet q;
  vector<unsigned long> r(row, row + nnz), c(col, col + nnz);
  vector<float> vf;
  vector<double> vd;
  if (val_dtype == FLOAT) vf.assign(val, val + nnz);
  else vd.assign(val, val + nnz);
  RefMatrix *h = new RefMatrix();
  h->m = init_sparse_struct_by_coo_vector(r, c, vf, vd, (data_type)val_dtype, cols - 1, rows - 1);
  h->op = init_op_manager(h->m);
  return h;
}

// long_short_row_decomposition frees the matrix it is given (op_manager.cc:120): the handle `hv` is empty
// afterwards and must not be used again.
int64_t ref_matrix_long_short_row_decomposition(void *hv, const uint64_t *low_bounds, uint64_t n_bounds, void **parts,
                                                uint64_t cap) {
  Quiet q;
  RefMatrix *h = (RefMatrix *)hv;
  vector<unsigned int> b(low_bounds, low_bounds + n_bounds);
  vector<sparse_struct_t *> out = long_short_row_decomposition(h->m, b);
  h->m = NULL;
  h->op->matrix = NULL;
  if (out.size() > cap) return -1;
  for (size_t i = 0; i < out.size(); i++) {
    RefMatrix *p = new RefMatrix();
    p->m = out[i];
    p->op = init_op_manager(out[i]);
    parts[i] = p;
  }
  return (int64_t)out.size();
}

// total_row_level_padding* and dense_col_level_padding (op_manager.cc:5361, :5221, :5043; op_manager.hpp:221)
int ref_matrix_total_row_level_padding(void *hv, uint64_t multiple, int position, uint64_t input_col_index) {
  Quiet q;
  total_row_level_padding(((RefMatrix *)hv)->op, multiple, (global_padding_position)position, input_col_index);
  return 0;
}

int ref_matrix_total_row_level_padding_direct(void *hv, uint64_t target_size, unsigned padding_col_num, int position,
                                              uint64_t input_col_index) {
  Quiet q;
  total_row_level_padding_direct(((RefMatrix *)hv)->op, target_size, padding_col_num,
                                 (global_padding_position)position, input_col_index);
  return 0;
}

int ref_matrix_total_row_level_padding_add(void *hv, uint64_t add_size, unsigned padding_col_num, int position,
                                           uint64_t input_col_index) {
  Quiet q;
  total_row_level_padding_add(((RefMatrix *)hv)->op, add_size, padding_col_num, (global_padding_position)position,
                              input_col_index);
  return 0;
}

int ref_matrix_dense_col_level_padding(void *hv, const uint64_t *row_index, const uint64_t *padding_target_size,
                                       uint64_t n) {
  Quiet q;
  dense_col_level_padding(((RefMatrix *)hv)->op, NULL, vector<unsigned long>(row_index, row_index + n),
                          vector<unsigned long>(padding_target_size, padding_target_size + n));
  return 0;
}

int ref_execute_node(void *hv, int node_type, int64_t sub, const long *scalars, int n_scalars, const uint64_t *list,
                     uint64_t n_list, const uint64_t *counts, uint64_t n_counts) {
  Quiet q;
  RefMatrix *h = (RefMatrix *)hv;
  exe_node_t node;
  node.type = (exe_node_type)node_type;
  vector<vector<unsigned int>> nested;
  uint64_t k = 0;
  for (uint64_t i = 0; i < n_counts; i++) {
    vector<unsigned int> v;
    for (uint64_t j = 0; j < counts[i]; j++) v.push_back((unsigned int)list[k++]);
    nested.push_back(v);
  }
  switch (node.type) {
    case DENSE_ROW_COARSE_SORT: {
      total_dense_block_coarse_sort(h->op, vector<unsigned long>(list, list + n_list));
      return 0;
    }
    case DENSE_ROW_DIV: {
      // scalars {sub-block, strip height} and no list: strips of equal height inside a sub-block of an already
      // divided matrix, fixed_len_row_div(matrix, sub_block, len) (op_manager.cc:243-365; upstream's var_len_row_div
      // stops at a sub-block, :520)
      if (n_list == 0 && n_scalars >= 2) {
        fixed_len_row_div(h->m, h->m->block_coor_table.item_arr[scalars[0]], (int)scalars[1]);
        return 0;
      }
      vector<unsigned long> pos(list, list + n_list);
      if (pos.size() <= 2) return 0;
      var_len_row_div(h->m, NULL, pos);
      return 0;
    }
    case DENSE_FINE_SORT:
      if (n_list == 0) total_dense_block_sort(h->op);
      else total_dense_block_sort(h->op, vector<unsigned long>(list, list + n_list));
      return 0;
    case DENSE_FIXED_COL_DIV:  // exe_graph.cc:1615-1640: the whole matrix first, a sub-block of the table afterwards
      if (h->m->block_coor_table.item_arr.size() == 0) fixed_len_col_div(h->m, NULL, (int)scalars[0]);
      else fixed_len_col_div(h->m, h->m->block_coor_table.item_arr[n_scalars >= 2 ? scalars[1] : 0], (int)scalars[0]);
      return 0;
    case COMPRESS:
      compress_dense_view(h->m);
      return 0;
    case COMPRESSED_BLOCK_SORT: {
      // upstream has the operator (op_manager.cc:4104) but no node executor for it; its templates insist on
      // compressed_block_t::is_sorted (e.g. direct_atom_op.cc:156), which the operator leaves to its caller
      compressed_block_t *cb = h->m->block_coor_table.item_arr[sub]->compressed_block_ptr;
      vector<unsigned long> blocks(list, list + n_list);
      if (blocks.empty())
        for (unsigned long b = 0; b < cb->read_index[2]->block_num; b++) blocks.push_back(b);
      compressed_block_sort(cb, blocks);
      cb->is_sorted = true;
      return 0;
    }
    case COMPRESSED_ROW_PADDING: {
      exe_compress_row_padding_param_t p;
      p.multiply = scalars[0];
      p.padding_row_length = scalars[1];
      node.param = &p;
      execute_exe_compress_row_padding_node(h->m, node, sub);
      return 0;
    }
    case COMPRESSED_THREAD_LEVEL_NNZ_DIV: {
      exe_compress_thread_level_nnz_div_param_t p;
      p.TLB_nnz_num = scalars[0];
      node.param = &p;
      execute_exe_compress_thread_level_nnz_div_node(h->m, node, sub);
      return 0;
    }
    case COMPRESSED_THREAD_LEVEL_COL_DIV: {
      exe_compress_thread_level_col_div_param_t p;
      p.col_num_of_TLB_in_each_parent_block.assign(list, list + n_list);
      node.param = &p;
      execute_exe_compress_TLB_col_div_node(h->m, node, sub);
      return 0;
    }
    case COMPRESSED_THREAD_LEVEL_ROW_DIV: {
      exe_compress_thread_level_row_div_param_t p;
      node.param = &p;
      execute_exe_compress_TLB_row_div_node(h->m, node, sub);
      return 0;
    }
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV: {
      exe_compress_tblock_level_row_div_param_t p;
      for (uint64_t i = 0; i < n_list; i++) p.row_num_of_each_BLB.push_back((unsigned int)list[i]);
      node.param = &p;
      execute_exe_compress_BLB_row_div_node(h->m, node, sub);
      return 0;
    }
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV: {
      exe_compress_tblock_level_col_div_param_t p;
      p.col_block_nnz_num_of_each_BLB = nested;
      node.param = &p;
      execute_exe_compress_BLB_col_div_node(h->m, node, sub);
      return 0;
    }
    case COMPRESSED_WARP_LEVEL_ROW_DIV: {
      exe_compress_warp_level_row_div_param_t p;
      p.row_num_of_each_WLB_in_BLB = nested;
      node.param = &p;
      execute_exe_compress_WLB_row_div_node(h->m, node, sub);
      return 0;
    }
    case COMPRESSED_WARP_LEVEL_COL_DIV: {
      exe_compress_warp_level_col_div_param_t p;
      p.col_num_of_WLB_in_each_parent_row_block_or_BLB = nested;
      node.param = &p;
      execute_exe_compress_WLB_col_div_node(h->m, node, sub);
      return 0;
    }
    default:
      return -1;
  }
}

// strategy -> node parameters (upstream execute_*_param_strategy) -> node
int ref_execute_strategy(void *hv, int strategy, int64_t sub, const long p[4]) {
  Quiet q;
  RefMatrix *h = (RefMatrix *)hv;
  exe_node_t node;
  switch ((exe_node_param_set_strategy)strategy) {
    case COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY: {
      compressed_row_padding_direct_param_strategy_t s;
      s.multiply = p[0]; s.padding_row_length = p[1];
      exe_compress_row_padding_param_t param;
      execute_compressed_row_padding_direct_param_strategy(&s, &param, h->m, sub);
      node.type = COMPRESSED_ROW_PADDING; node.param = &param;
      execute_exe_node_in_compressed_sub_matrix(h->m, sub, node);
      return 0;
    }
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY: {
      compressed_tblock_level_row_div_evenly_param_strategy_t s;
      s.block_row_num = p[0];
      exe_compress_tblock_level_row_div_param_t param;
      execute_compressed_tblock_level_row_div_evenly_param_strategy(&s, &param, h->m, sub);
      node.type = COMPRESSED_TBLOCK_LEVEL_ROW_DIV; node.param = &param;
      execute_exe_node_in_compressed_sub_matrix(h->m, sub, node);
      return 0;
    }
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY: {
      compressed_tblock_level_row_div_acc_to_least_nnz_param_strategy_t s;
      s.nnz_low_bound = p[0];
      exe_compress_tblock_level_row_div_param_t param;
      execute_compressed_tblock_level_row_div_acc_to_least_nnz_param_strategy(&s, &param, h->m, sub);
      node.type = COMPRESSED_TBLOCK_LEVEL_ROW_DIV; node.param = &param;
      execute_exe_node_in_compressed_sub_matrix(h->m, sub, node);
      return 0;
    }
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: {
      compressed_tblock_level_col_div_fixed_param_strategy_t s;
      s.col_block_nnz_num = p[0];
      exe_compress_tblock_level_col_div_param_t param;
      execute_compressed_tblock_level_col_div_fixed_param_strategy(&s, &param, h->m, sub);
      node.type = COMPRESSED_TBLOCK_LEVEL_COL_DIV; node.param = &param;
      execute_exe_node_in_compressed_sub_matrix(h->m, sub, node);
      return 0;
    }
    case COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY: {
      compressed_warp_level_row_div_evenly_param_strategy_t s;
      s.warp_row_num_of_each_BLB = p[0];
      exe_compress_warp_level_row_div_param_t param;
      execute_compressed_warp_level_row_div_evenly_param_strategy(&s, &param, h->m, sub);
      node.type = COMPRESSED_WARP_LEVEL_ROW_DIV; node.param = &param;
      execute_exe_node_in_compressed_sub_matrix(h->m, sub, node);
      return 0;
    }
    case COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: {
      compressed_warp_level_col_div_fixed_param_strategy_t s;
      s.col_block_nnz_num = p[0];
      exe_compress_warp_level_col_div_param_t param;
      execute_compressed_warp_level_col_div_fixed_param_strategy(&s, &param, h->m, sub);
      node.type = COMPRESSED_WARP_LEVEL_COL_DIV; node.param = &param;
      execute_exe_node_in_compressed_sub_matrix(h->m, sub, node);
      return 0;
    }
    case COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY: {
      compressed_thread_level_row_div_none_param_strategy_t s;
      exe_compress_thread_level_row_div_param_t param;
      execute_compressed_thread_level_row_div_none_param_strategy(&s, &param, h->m, sub);
      node.type = COMPRESSED_THREAD_LEVEL_ROW_DIV; node.param = &param;
      execute_exe_node_in_compressed_sub_matrix(h->m, sub, node);
      return 0;
    }
    case COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: {
      compressed_thread_level_col_div_fixed_param_strategy_t s;
      s.col_block_nnz_num = p[0];
      exe_compress_thread_level_col_div_param_t param;
      execute_compressed_thread_level_col_div_fixed_param_strategy(&s, &param, h->m, sub);
      node.type = COMPRESSED_THREAD_LEVEL_COL_DIV; node.param = &param;
      execute_exe_node_in_compressed_sub_matrix(h->m, sub, node);
      return 0;
    }
    case COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT_PARAM_STRATEGY: {
      compressed_thread_level_nnz_div_direct_param_strategy_t s;
      s.block_nnz_num = p[0];
      exe_compress_thread_level_nnz_div_param_t param;
      execute_compressed_thread_level_nnz_div_direct_param_strategy(&s, &param, h->m, sub);
      node.type = COMPRESSED_THREAD_LEVEL_NNZ_DIV; node.param = &param;
      execute_exe_node_in_compressed_sub_matrix(h->m, sub, node);
      return 0;
    }
    case DENSE_ROW_COARSE_SORT_FIXED_PARAM_STRATEGY: {
      dense_row_coarse_sort_fixed_param_strategy_t s;
      s.row_nnz_low_bound_step_size = p[0];
      exe_dense_row_coarse_sort_param_t param;
      execute_dense_row_coarse_sort_fixed_param_strategy(&s, &param, h->m);
      total_dense_block_coarse_sort(h->op, param.bin_row_nnz_low_bound);
      return 0;
    }
    case DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ_PARAM_STRATEGY: {
      dense_row_div_acc_to_exponential_increase_row_nnz_param_strategy_t s;
      s.lowest_nnz_bound_of_row = p[0]; s.highest_nnz_bound_of_row = p[1]; s.expansion_rate = p[2]; s.sub_dense_block_id = p[3];
      exe_dense_row_div_param_t param;
      execute_dense_row_div_acc_to_exponential_increase_row_nnz_param_strategy(&s, &param, h->m);
      if (param.row_div_position.size() > 2) var_len_row_div(h->m, NULL, param.row_div_position);
      return 0;
    }
    case COMPRESS_NONE_PARAM_STRATEGY:
      compress_dense_view(h->m);
      return 0;
    default:
      return -1;
  }
}

int ref_complete_blocking(void *hv, int64_t sub) {
  Quiet q;
  RefMatrix *h = (RefMatrix *)hv;
  execute_default_div_to_complete_each_level_blocking(h->m, sub);
  return 0;
}

int ref_matrix_info(void *hv, uint64_t out[8]) {
  RefMatrix *h = (RefMatrix *)hv;
  out[0] = h->m->dense_row_number; out[1] = h->m->dense_col_number; out[2] = h->m->nnz; out[3] = h->m->origin_nnz;
  out[4] = h->m->block_coor_table.item_arr.size(); out[5] = h->m->is_sorted; out[6] = h->m->is_compressed; out[7] = 32;
  return 0;
}

int64_t ref_get_u64(void *hv, int64_t sub, int slot, int field, uint64_t *out, uint64_t cap, int *dtype) {
  RefMatrix *h = (RefMatrix *)hv;
  sparse_struct_t *m = h->m;
  if (slot == 100) return put(m->sorted_row_index, m->data_type_of_sorted_row_index, m->dense_row_number, out, cap, dtype);
  if (slot == 103) return put(field == 0 ? m->coo_row_index_cache : m->coo_col_index_cache, UNSIGNED_LONG, m->nnz, out, cap, dtype);
  if (sub < 0 || (uint64_t)sub >= m->block_coor_table.item_arr.size()) return -2;
  dense_block_table_item_t *it = m->block_coor_table.item_arr[sub];
  if (slot == 101) {
    uint64_t v[7] = {it->min_dense_row_index, it->max_dense_row_index, it->min_dense_col_index, it->max_dense_col_index,
                     it->begin_coo_index, it->end_coo_index, it->is_col_blocked};
    return put(v, UNSIGNED_LONG, 7, out, cap, dtype);
  }
  compressed_block_t *cb = it->compressed_block_ptr;
  if (cb == NULL) return -2;
  if (slot == 104) {  // y_write_index[0] of compressed_block_sort
    if (cb->y_write_index.empty()) return -1;
    return put(cb->y_write_index[0]->index_arr, cb->y_write_index[0]->index_data_type, cb->y_write_index[0]->length, out, cap, dtype);
  }
  if (slot == 102) {
    uint64_t v[4] = {cb->share_row_with_other_block, cb->share_row_with_other_warp, cb->share_row_with_other_thread,
                     cb->read_index.size()};
    return put(v, UNSIGNED_LONG, 4, out, cap, dtype);
  }
  if (slot < 0 || slot >= 7) return -2;
  if ((size_t)slot >= cb->read_index.size()) return -1;
  index_of_compress_block_t *ix = cb->read_index[slot];
  bool is_tlb = ix->level_of_this_index == THREAD_LEVEL;
  bool is_wlb = ix->level_of_this_index == WRAP_LEVEL;
  uint64_t wlb_num = cb->read_index.size() > 3 ? cb->read_index[3]->block_num : 0;
  switch (field) {
    case 0:  // index_arr: COO payload has `length` entries, CSR offsets block_num + 1
      return put(ix->index_arr, ix->index_data_type,
                 ix->index_compressed_type == COO ? ix->length : ix->block_num + 1, out, cap, dtype);
    case 1: return put(ix->index_of_the_first_row_arr, ix->data_type_of_index_of_the_first_row_arr, ix->block_num, out, cap, dtype);
    case 2: return put(ix->row_number_of_block_arr, ix->data_type_of_row_number_of_block_arr, ix->block_num, out, cap, dtype);
    case 3:  // BLB: block_num + 1 offsets; WLB: block_num
      return put(ix->coo_begin_index_arr, ix->data_type_of_coo_begin_index_arr, is_wlb ? ix->block_num : ix->block_num + 1, out, cap, dtype);
    case 4:  // TLB level stores one size per WLB
      return put(ix->coo_block_size_arr, ix->data_type_of_coo_block_size_arr, is_tlb ? wlb_num : ix->block_num, out, cap, dtype);
    case 5: {
      // `length` of the TLB level is never initialised upstream -> reported as 0
      uint64_t v[9] = {ix->block_num, is_tlb ? 0 : ix->length, ix->max_row_index, ix->min_row_index, ix->max_col_index,
                       ix->min_col_index, (uint64_t)ix->level_of_this_index, (uint64_t)ix->index_compressed_type,
                       (uint64_t)ix->type_of_index};
      return put(v, UNSIGNED_LONG, 9, out, cap, dtype);
    }
    default: return -2;
  }
}

int64_t ref_get_f64(void *hv, int64_t sub, int which, double *out, uint64_t cap) {
  RefMatrix *h = (RefMatrix *)hv;
  sparse_struct_t *m = h->m;
  void *arr = NULL;
  uint64_t n = 0;
  data_type dt = m->val_data_type;
  if (which == 3) { arr = m->coo_value_cache; n = m->nnz; }
  else {
    if (sub < 0 || (uint64_t)sub >= m->block_coor_table.item_arr.size()) return -2;
    compressed_block_t *cb = m->block_coor_table.item_arr[sub]->compressed_block_ptr;
    if (cb == NULL) return -2;
    if (which == 0) { arr = cb->val_arr; n = cb->size; }
    if (which == 1) { arr = cb->padding_val_arr; n = cb->padding_arr_size; }
    if (which == 2) { arr = cb->staggered_padding_val_arr; n = cb->staggered_padding_val_arr_size; }
  }
  if (arr == NULL) return -1;
  if (out)
    for (uint64_t i = 0; i < n && i < cap; i++) out[i] = read_double_from_array_with_data_type(arr, dt, i);
  return (int64_t)n;
}

}  // extern "C"

// ---------------------------------------------------------------------------
// Kernel templates: upstream init_<T>_template + try_all_compress, dumped by name.
namespace {
struct NamedArr { const char *name; void *ptr; data_type dt; uint64_t n; int compress; };
struct TplView {
  std::vector<NamedArr> arrs;
  std::vector<std::pair<const char *, uint64_t>> scalars;
  void *val = NULL; data_type val_dt = FLOAT; uint64_t val_n = 0;
};
#define ARR(T, field, cfield) v.arrs.push_back({#field, (T)->field, (T)->data_type_of_##field, (T)->size_of_##field, (int)(T)->cfield})
#define ARRN(T, field) v.arrs.push_back({#field, (T)->field, (T)->data_type_of_##field, (T)->size_of_##field, 0})
#define COMMON(T)                                                                                   \
  v.scalars.push_back({"kernal_first_row_index", (T)->kernal_first_row_index});                     \
  v.scalars.push_back({"kernal_first_col_index", (T)->kernal_first_col_index});                     \
  v.scalars.push_back({"global_sort_index", (uint64_t)(T)->global_sort_index});                     \
  v.scalars.push_back({"local_sort_index", (uint64_t)(T)->local_sort_index});                       \
  ARRN(T, col_index_arr);                                                                           \
  v.val = (T)->val_arr; v.val_dt = (T)->data_type_of_val_arr; v.val_n = (T)->size_of_val_arr;

TplView view_of(void *tp, template_type type) {
  TplView v;
  switch (type) {
    case DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS: {
      auto *t = (direct_atom_template_warp_block_compress_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_atom_add});
      v.scalars.push_back({"effective_TLB_num", t->effective_TLB_num});
      v.scalars.push_back({"thread_block_size_in_block", t->thread_block_size_in_block});
      ARR(t, global_row_index_of_thread_level_block, global_row_index_compress);
      break;
    }
    case DIRECT_ATOM_TEMPLATE_WARP_COMPRESS: {
      auto *t = (direct_atom_template_warp_compress_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_atom_add});
      v.scalars.push_back({"effective_TLB_num", t->effective_TLB_num});
      ARR(t, global_row_index_of_thread_level_block, global_row_index_compress);
      ARR(t, block_begin_thread_index_offset, block_begin_thread_index_offset_compress);
      ARR(t, block_nz_begin_offset, block_nz_begin_offset_compress);
      ARR(t, thread_block_size_in_block, thread_block_size_in_block_compress);
      break;
    }
    case SHARED_MEMORY_LONG_ROW_TEMPLATE: {
      auto *t = (shared_memory_long_row_template_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_atom_add});
      ARR(t, row_index_of_block_level_block, row_index_of_block_level_block_compress);
      ARR(t, block_nz_begin_offset, block_nz_begin_offset_compress);
      break;
    }
    case DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE: {
      auto *t = (direct_atom_total_warp_reduce_template_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_atom_add});
      v.scalars.push_back({"effective_WLB_num", t->effective_WLB_num});
      ARR(t, global_row_index_of_warp_level_block, global_row_index_of_warp_level_block_compress);
      ARR(t, global_warp_nz_begin_offset, global_warp_nz_begin_offset_compress);
      break;
    }
    case SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE: {
      auto *t = (shared_memory_total_warp_reduce_template_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_atom_add});
      v.scalars.push_back({"effective_row_num", t->effective_row_num});
      ARR(t, row_offset_in_warp_tmp_result, row_offset_in_warp_tmp_result_compress);
      ARR(t, block_first_row_index, block_first_row_index_compress);
      ARR(t, block_begin_warp_index_offset, block_begin_warp_index_offset_compress);
      ARR(t, global_warp_block_first_nz, global_warp_block_first_nz_compress);
      break;
    }
    case SHARED_MEMORY_TEMPLATE_WARP_COMPRESS: {
      auto *t = (shared_memory_template_warp_compress_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_atom_add});
      v.scalars.push_back({"effective_row_num", t->effective_row_num});
      ARR(t, row_offset_in_thread_tmp_result, row_offset_in_thread_tmp_result_compress);
      ARR(t, block_first_row_index, block_first_row_index_compress);
      ARR(t, block_begin_thread_index_offset, block_begin_thread_index_offset_compress);
      ARR(t, thread_block_size_in_block, thread_block_size_in_block_compress);
      ARR(t, block_nz_begin_offset, block_nz_begin_offset_compress);
      break;
    }
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE: {
      auto *t = (unaligned_warp_reduce_same_TLB_size_template_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_all_force_atom_add});
      v.scalars.push_back({"global_thread_level_block_size", t->global_thread_level_block_size});
      v.scalars.push_back({"bit_num_of_thread_level_combine_meta", (uint64_t)t->bit_num_of_thread_level_combine_meta});
      v.scalars.push_back({"bit_num_of_sum_begin_bit_flag", (uint64_t)t->bit_num_of_sum_begin_bit_flag});
      v.scalars.push_back({"bit_num_of_first_relative_reduce_row_of_thread_level_block", (uint64_t)t->bit_num_of_first_relative_reduce_row_of_thread_level_block});
      v.scalars.push_back({"bit_num_of_tmp_result_reduce_offset_of_thread_level_block", (uint64_t)t->bit_num_of_tmp_result_reduce_offset_of_thread_level_block});
      ARR(t, global_first_row_index_of_warp_level_block, global_first_row_index_of_warp_level_block_compress);
      ARRN(t, combine_meta_of_thread_level_block);
      ARRN(t, first_relative_reduce_row_of_thread_level_block);
      ARRN(t, tmp_result_reduce_offset_of_thread_level_block);
      break;
    }
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE: {
      auto *t = (unaligned_warp_reduce_same_TLB_size_template_with_warp_reduce_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_all_force_atom_add});
      v.scalars.push_back({"global_thread_level_block_size", t->global_thread_level_block_size});
      v.scalars.push_back({"bit_num_of_thread_level_combine_meta", (uint64_t)t->bit_num_of_thread_level_combine_meta});
      ARR(t, global_first_row_index_of_warp_level_block, global_first_row_index_of_warp_level_block_compress);
      ARRN(t, combine_meta_of_thread_level_block);
      ARRN(t, first_relative_reduce_row_of_thread_level_block);
      ARRN(t, tmp_result_reduce_offset_of_thread_level_block);
      break;
    }
    case DIRECT_ATOM_TEMPLATE: {
      auto *t = (direct_atom_template_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_atom_add});
      ARR(t, global_row_index_of_thread_level_block, global_row_index_compress);
      ARR(t, block_begin_warp_index_offset, block_begin_warp_index_compress);
      ARR(t, warp_begin_thread_index_offset, warp_begin_thread_index_compress);
      ARR(t, thread_block_size_in_warp, thread_block_size_compress);
      ARR(t, block_nz_begin_offset, block_nz_begin_offset_compress);
      ARR(t, warp_nz_begin_offset, warp_nz_begin_offset_compress);
      break;
    }
    case SHARED_MEMORY_TEMPLATE: {
      auto *t = (shared_memory_template_t *)tp;
      COMMON(t)
      v.scalars.push_back({"is_atom_add", (uint64_t)t->is_atom_add});
      ARR(t, row_offset_in_thread_tmp_result, row_offset_in_thread_tmp_result_compress);
      ARR(t, block_first_row_index, block_first_row_index_compress);
      ARR(t, block_begin_warp_index_offset, block_begin_warp_index_offset_compress);
      ARR(t, warp_begin_thread_index_offset, warp_begin_thread_index_offset_compress);
      ARR(t, thread_block_size_in_warp, thread_block_size_in_warp_compress);
      ARR(t, block_nz_begin_offset, block_nz_begin_offset_compress);
      ARR(t, warp_nz_begin_offset, warp_nz_begin_offset_compress);
      break;
    }
    default: break;
  }
  return v;
}
}  // namespace

extern "C" {

// 1 supported / 0 not (upstream is_supported_by_<T>(matrix, sub))
int ref_template_is_supported(void *hv, int64_t sub, int type) {
  Quiet q;
  RefMatrix *h = (RefMatrix *)hv;
  switch ((template_type)type) {
    case DIRECT_ATOM_TEMPLATE: {
      // the builder overload (direct_atom_op.cc:257-287) only adds "no row padding" to the matrix overload
      dense_block_table_item_t *it = h->m->block_coor_table.item_arr[sub];
      for (int lvl = 0; lvl < 4; lvl++)
        if (it->max_dense_row_index != it->compressed_block_ptr->read_index[lvl]->max_row_index) return 0;
      return is_supported_by_direct_atom_template(h->m, sub);
    }
    case SHARED_MEMORY_TEMPLATE: return is_supported_by_shared_memory_template(h->m, sub);
    case DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS: return is_supported_by_direct_atom_template_warp_block_compress(h->m, sub);
    case DIRECT_ATOM_TEMPLATE_WARP_COMPRESS: return is_supported_by_direct_atom_template_warp_compress(h->m, sub);
    case SHARED_MEMORY_LONG_ROW_TEMPLATE: return is_supported_by_shared_memory_long_row_template(h->m, sub);
    case DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE: return is_supported_by_direct_atom_total_warp_reduce_template(h->m, sub);
    case SHARED_MEMORY_TEMPLATE_WARP_COMPRESS: return is_supported_by_shared_memory_template_warp_compress(h->m, sub);
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE: return is_supported_by_unaligned_warp_reduce_same_TLB_size_template(h->m, sub);
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE: return is_supported_by_unaligned_warp_reduce_same_TLB_size_template_with_warp_reduce(h->m, sub);
    default: return -1;  // SHARED_MEMORY_TOTAL_WARP_REDUCE: upstream's matrix overload always trips its own assert
  }
}

int ref_template_init(void *hv, int64_t sub, int type, int compress) {
  Quiet q;
  RefMatrix *h = (RefMatrix *)hv;
  if (h->builder == NULL) {
    h->builder = init_code_builder(h->op);
    h->templates.assign(h->m->block_coor_table.item_arr.size(), (void *)NULL);
    h->template_types.assign(h->m->block_coor_table.item_arr.size(), NONE_TEMPLATE);
  }
  void *t = NULL;
  switch ((template_type)type) {
    case DIRECT_ATOM_TEMPLATE: { auto *p = init_direct_atom_template(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    case SHARED_MEMORY_TEMPLATE: { auto *p = init_shared_memory_template(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    case DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS: { auto *p = init_direct_atom_template_warp_block_compress(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    case DIRECT_ATOM_TEMPLATE_WARP_COMPRESS: { auto *p = init_direct_atom_template_warp_compress(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    case SHARED_MEMORY_LONG_ROW_TEMPLATE: { auto *p = init_shared_memory_long_row_template(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    case DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE: { auto *p = init_direct_atom_total_warp_reduce_template(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    case SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE: { auto *p = init_shared_memory_total_warp_reduce_template(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    case SHARED_MEMORY_TEMPLATE_WARP_COMPRESS: { auto *p = init_shared_memory_template_warp_compress(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE: { auto *p = init_unaligned_warp_reduce_same_TLB_size_template(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE: { auto *p = init_unaligned_warp_reduce_same_TLB_size_template_with_warp_reduce(h->builder, sub); if (compress) try_all_compress(p); t = p; break; }
    default: return -1;
  }
  h->templates[sub] = t;
  h->template_types[sub] = (template_type)type;
  return 0;
}

int64_t ref_template_get_u64(void *hv, int64_t sub, const char *name, uint64_t *out, uint64_t cap, int *dtype, int *compress) {
  RefMatrix *h = (RefMatrix *)hv;
  TplView v = view_of(h->templates[sub], h->template_types[sub]);
  for (auto &a : v.arrs)
    if (!strcmp(a.name, name)) {
      if (compress) *compress = a.compress;
      return put(a.ptr, a.dt, a.n, out, cap, dtype);
    }
  return -1;
}

int64_t ref_template_get_f64(void *hv, int64_t sub, double *out, uint64_t cap) {
  RefMatrix *h = (RefMatrix *)hv;
  TplView v = view_of(h->templates[sub], h->template_types[sub]);
  if (out)
    for (uint64_t i = 0; i < v.val_n && i < cap; i++) out[i] = read_double_from_array_with_data_type(v.val, v.val_dt, i);
  return (int64_t)v.val_n;
}

// "name=value\n" for every scalar, "array:name\n" for every array
int64_t ref_template_describe(void *hv, int64_t sub, char *out, uint64_t cap) {
  RefMatrix *h = (RefMatrix *)hv;
  TplView v = view_of(h->templates[sub], h->template_types[sub]);
  std::string s;
  for (auto &kv : v.scalars) s += std::string(kv.first) + "=" + std::to_string(kv.second) + "\n";
  for (auto &a : v.arrs) s += std::string("array:") + a.name + "\n";
  if (out && cap) { strncpy(out, s.c_str(), cap - 1); out[cap - 1] = 0; }
  return (int64_t)s.size();
}

// ---- search control and report text -----------------------------------------------------------
// every combination an upstream enumerator over n integer knobs yields, row-major in `out`
// (set_param_combination_to_next, param_enumerater.cc:199); returns the number of combinations
int64_t ref_selftest_param_enumerator(int n, const long *low, const long *up, const long *step, long *out, uint64_t cap) {
  Quiet q;
  std::vector<long> knob(n);
  param_enumerater_t e;
  for (int i = 0; i < n; i++) register_integer_independ_param_to_enumerater(&e, &knob[i], low[i], up[i], step[i]);
  int64_t count = 0;
  while (set_param_combination_to_next(&e) == false) {
    for (int i = 0; i < n; i++)
      if ((uint64_t)(count * n + i) < cap) out[count * n + i] = knob[i];
    count++;
  }
  return count;
}

// continue_search(strategy, gflops) for a series of candidate results, no time limit
// (search_strategy.cc:24-81); go[i] = its answer after candidate i
int ref_selftest_search_strategy(uint64_t struggle, const float *gflops, int n, int *go) {
  Quiet q;
  search_strategy_t s = init_search_strategy(struggle, 1e9);
  for (int i = 0; i < n; i++) go[i] = continue_search(&s, gflops[i]) ? 1 : 0;
  return 0;
}

static int64_t put_text(const std::string &s, char *out, uint64_t cap) {
  if (out && cap) { strncpy(out, s.c_str(), cap - 1); out[cap - 1] = 0; }
  return (int64_t)s.size();
}

// convert_stategy_node_to_string (parameter_set_strategy.cc:1309) of one strategy node with knobs p
int64_t ref_strategy_report(int strategy, const long p[4], char *out, uint64_t cap) {
  Quiet q;
  param_strategy_node_t node;
  int dummy = 0;
  node.param = &dummy;  // only checked for non-NULL
  node.strategy_type = (exe_node_param_set_strategy)strategy;
  compressed_row_padding_direct_param_strategy_t s0;
  compressed_tblock_level_row_div_evenly_param_strategy_t s1;
  compressed_tblock_level_row_div_acc_to_least_nnz_param_strategy_t s2;
  compressed_tblock_level_col_div_fixed_param_strategy_t s3;
  compressed_warp_level_row_div_evenly_param_strategy_t s4;
  compressed_warp_level_col_div_fixed_param_strategy_t s5;
  compressed_thread_level_row_div_none_param_strategy_t s6;
  compressed_thread_level_col_div_fixed_param_strategy_t s7;
  compressed_thread_level_nnz_div_direct_param_strategy_t s8;
  dense_row_coarse_sort_fixed_param_strategy_t s9;
  compress_none_param_strategy_t s11;
  dense_row_div_acc_to_exponential_increase_row_nnz_param_strategy_t s12;
  switch (node.strategy_type) {
    case COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY: s0.multiply = p[0]; s0.padding_row_length = p[1]; node.param_strategy = &s0; node.node_type = COMPRESSED_ROW_PADDING; break;
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY: s1.block_row_num = p[0]; node.param_strategy = &s1; node.node_type = COMPRESSED_TBLOCK_LEVEL_ROW_DIV; break;
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY: s2.nnz_low_bound = p[0]; node.param_strategy = &s2; node.node_type = COMPRESSED_TBLOCK_LEVEL_ROW_DIV; break;
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: s3.col_block_nnz_num = p[0]; node.param_strategy = &s3; node.node_type = COMPRESSED_TBLOCK_LEVEL_COL_DIV; break;
    case COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY: s4.warp_row_num_of_each_BLB = p[0]; node.param_strategy = &s4; node.node_type = COMPRESSED_WARP_LEVEL_ROW_DIV; break;
    case COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: s5.col_block_nnz_num = p[0]; node.param_strategy = &s5; node.node_type = COMPRESSED_WARP_LEVEL_COL_DIV; break;
    case COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY: node.param_strategy = &s6; node.node_type = COMPRESSED_THREAD_LEVEL_ROW_DIV; break;
    case COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: s7.col_block_nnz_num = p[0]; node.param_strategy = &s7; node.node_type = COMPRESSED_THREAD_LEVEL_COL_DIV; break;
    case COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT_PARAM_STRATEGY: s8.block_nnz_num = p[0]; node.param_strategy = &s8; node.node_type = COMPRESSED_THREAD_LEVEL_NNZ_DIV; break;
    case DENSE_ROW_COARSE_SORT_FIXED_PARAM_STRATEGY: s9.row_nnz_low_bound_step_size = p[0]; node.param_strategy = &s9; node.node_type = DENSE_ROW_COARSE_SORT; break;
    case COMPRESS_NONE_PARAM_STRATEGY: node.param_strategy = &s11; node.node_type = COMPRESS; break;
    case DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ_PARAM_STRATEGY:
      s12.lowest_nnz_bound_of_row = p[0]; s12.highest_nnz_bound_of_row = p[1]; s12.expansion_rate = p[2]; s12.sub_dense_block_id = p[3];
      node.param_strategy = &s12; node.node_type = DENSE_ROW_DIV; break;
    default: return -1;
  }
  return put_text(convert_stategy_node_to_string(node), out, cap);
}

// convert_template_node_to_string (exe_graph.cc:3317) for a template type with the given launch parameters
int64_t ref_template_node_report(int type, long tblock_num, long thread_num_in_block, long thread_num_of_row_reduce, char *out,
                                 uint64_t cap) {
  Quiet q;
  template_node_t node;
  node.type = (template_type)type;
  long two[2] = {tblock_num, thread_num_in_block};                              // {tblock_num, thread_num_in_block}
  long three[3] = {tblock_num, thread_num_in_block, thread_num_of_row_reduce};  // + thread_num_of_row_reduce
  long one[1] = {thread_num_in_block};
  switch (node.type) {
    case SHARED_MEMORY_TEMPLATE: case SHARED_MEMORY_TEMPLATE_WARP_COMPRESS: case SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE:
      node.template_param = three; break;
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE: node.template_param = one; break;
    default: node.template_param = two;
  }
  return put_text(convert_template_node_to_string(&node), out, cap);
}

}  // extern "C"

// ---- the assembled report of a whole graph ------------------------------------------------------
namespace {
// a strategy with its knobs as the upstream parameter struct (heap: the graph keeps pointers; a test process ends soon)
struct StrategyParam { exe_node_type node; void *param; };
StrategyParam strategy_param(int strategy, const long *p) {
  switch ((exe_node_param_set_strategy)strategy) {
    case COMPRESSED_ROW_PADDING_DIRECT_PARAM_STRATEGY: { auto *s = new compressed_row_padding_direct_param_strategy_t(); s->multiply = p[0]; s->padding_row_length = p[1]; return {COMPRESSED_ROW_PADDING, s}; }
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY: { auto *s = new compressed_tblock_level_row_div_evenly_param_strategy_t(); s->block_row_num = p[0]; return {COMPRESSED_TBLOCK_LEVEL_ROW_DIV, s}; }
    case COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ_PARAM_STRATEGY: { auto *s = new compressed_tblock_level_row_div_acc_to_least_nnz_param_strategy_t(); s->nnz_low_bound = p[0]; return {COMPRESSED_TBLOCK_LEVEL_ROW_DIV, s}; }
    case COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: { auto *s = new compressed_tblock_level_col_div_fixed_param_strategy_t(); s->col_block_nnz_num = p[0]; return {COMPRESSED_TBLOCK_LEVEL_COL_DIV, s}; }
    case COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY_PARAM_STRATEGY: { auto *s = new compressed_warp_level_row_div_evenly_param_strategy_t(); s->warp_row_num_of_each_BLB = p[0]; return {COMPRESSED_WARP_LEVEL_ROW_DIV, s}; }
    case COMPRESSED_WARP_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: { auto *s = new compressed_warp_level_col_div_fixed_param_strategy_t(); s->col_block_nnz_num = p[0]; return {COMPRESSED_WARP_LEVEL_COL_DIV, s}; }
    case COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE_PARAM_STRATEGY: return {COMPRESSED_THREAD_LEVEL_ROW_DIV, new compressed_thread_level_row_div_none_param_strategy_t()};
    case COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED_PARAM_STRATEGY: { auto *s = new compressed_thread_level_col_div_fixed_param_strategy_t(); s->col_block_nnz_num = p[0]; return {COMPRESSED_THREAD_LEVEL_COL_DIV, s}; }
    case COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT_PARAM_STRATEGY: { auto *s = new compressed_thread_level_nnz_div_direct_param_strategy_t(); s->block_nnz_num = p[0]; return {COMPRESSED_THREAD_LEVEL_NNZ_DIV, s}; }
    case DENSE_ROW_COARSE_SORT_FIXED_PARAM_STRATEGY: { auto *s = new dense_row_coarse_sort_fixed_param_strategy_t(); s->row_nnz_low_bound_step_size = p[0]; return {DENSE_ROW_COARSE_SORT, s}; }
    case COMPRESS_NONE_PARAM_STRATEGY: return {COMPRESS, new compress_none_param_strategy_t()};
    case DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ_PARAM_STRATEGY: {
      auto *s = new dense_row_div_acc_to_exponential_increase_row_nnz_param_strategy_t();
      s->lowest_nnz_bound_of_row = p[0]; s->highest_nnz_bound_of_row = p[1]; s->expansion_rate = p[2]; s->sub_dense_block_id = p[3];
      return {DENSE_ROW_DIV, s};
    }
    case DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY: {
      // knobs: element count, value type, largest column index, largest row index; the elements themselves are
      // placeholders (row i % rows, column i % cols, value 1), the report prints only those four
      auto *s = new dense_begin_memory_cache_input_file_direct_param_strategy_t();
      s->val_data_type = (data_type)p[1];
      s->col_index_max = (unsigned long)p[2];
      s->row_index_max = (unsigned long)p[3];
      for (long i = 0; i < p[0]; i++) {
        s->row_index_cache.push_back((unsigned long)i % (s->row_index_max + 1));
        s->col_index_cache.push_back((unsigned long)i % (s->col_index_max + 1));
        if (s->val_data_type == DOUBLE) s->double_val_cache.push_back(1.0); else s->float_val_cache.push_back(1.0f);
      }
      return {BEGIN_MEMORY_CACHE_INPUT_FILE, s};
    }
    default: return {COMPRESS, NULL};
  }
}
}  // namespace

extern "C" {

// The report of a whole operator graph, assembled by upstream's own functions: the graph is built with
// add_a_exe_node_and_param_strategy_to_exe_dense_sub_graph / ..._compressed_sub_graph (default_auto_tuner.cc:2131, 2281),
// every sub-matrix gets its template node, and the text is what
// convert_dense_view_matrix_and_compressed_sub_block_exe_graph_and_template_to_string_safety
// (whilte_list_path_impl.cc:4150-4228) returns.  `desc` = n_dense, n_dense x (strategy, p0..p3), n_sub, then per
// sub-matrix: n_nodes, n_nodes x (strategy, p0..p3), template type, tblock_num, thread_num_in_block,
// thread_num_of_row_reduce.  with_frame != 0: the text main.cc:646-657 prints around it (the same stream
// insertions on the same float values) up to and including "finish search".
int64_t ref_graph_report(const long *desc, int64_t n_desc, int with_frame, float gflops, float time_ms, char *out, uint64_t cap) {
  std::string text;
  {
    Quiet q;
    int64_t at = 0;
    dense_view_matrix_and_compressed_sub_block_exe_graph_and_template_t graph;
    exe_dense_sub_graph_t &dense = graph.dense_sub_graph_and_param_strategy.dense_sub_graph;
    param_strategy_of_sub_graph_t &dense_strategy = graph.dense_sub_graph_and_param_strategy.dense_sub_graph_param_strategy;
    long n_dense = desc[at++];
    for (long i = 0; i < n_dense; i++, at += 5) {
      StrategyParam sp = strategy_param((int)desc[at], desc + at + 1);
      if (sp.param == NULL) return -1;
      add_a_exe_node_and_param_strategy_to_exe_dense_sub_graph(&dense, &dense_strategy, sp.node, (exe_node_param_set_strategy)desc[at], sp.param);
    }
    long n_sub = desc[at++];
    for (long s = 0; s < n_sub; s++) {
      compressed_sub_block_exe_graph_and_template_t sub;
      long n_nodes = desc[at++];
      for (long i = 0; i < n_nodes; i++, at += 5) {
        StrategyParam sp = strategy_param((int)desc[at], desc + at + 1);
        if (sp.param == NULL) return -1;
        add_a_exe_node_and_param_strategy_to_exe_compressed_sub_graph(&sub.sub_graph, &sub.sub_graph_param_strategy, sp.node, (exe_node_param_set_strategy)desc[at], sp.param);
      }
      sub.temp_node.type = (template_type)desc[at];
      long tblock = desc[at + 1], threads = desc[at + 2], row_reduce = desc[at + 3];
      at += 4;
      switch (sub.temp_node.type) {
        case DIRECT_ATOM_TEMPLATE: { auto *t = new direct_atom_template_node_param_t(); t->tblock_num = tblock; t->thread_num_in_block = threads; sub.temp_node.template_param = t; break; }
        case DIRECT_ATOM_TEMPLATE_WARP_COMPRESS: { auto *t = new direct_atom_template_warp_compress_node_param_t(); t->tblock_num = tblock; t->thread_num_in_block = threads; sub.temp_node.template_param = t; break; }
        case DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS: { auto *t = new direct_atom_template_warp_block_compress_node_param_t(); t->tblock_num = tblock; t->thread_num_in_block = threads; sub.temp_node.template_param = t; break; }
        case SHARED_MEMORY_TEMPLATE: { auto *t = new shared_memory_template_node_param_t(); t->tblock_num = tblock; t->thread_num_in_block = threads; t->thread_num_of_row_reduce = row_reduce; sub.temp_node.template_param = t; break; }
        case SHARED_MEMORY_TEMPLATE_WARP_COMPRESS: { auto *t = new shared_memory_template_warp_compress_node_param_t(); t->tblock_num = tblock; t->thread_num_in_block = threads; t->thread_num_of_row_reduce = row_reduce; sub.temp_node.template_param = t; break; }
        case SHARED_MEMORY_LONG_ROW_TEMPLATE: { auto *t = new shared_memory_long_row_template_node_param_t(); t->tblock_num = tblock; t->thread_num_in_block = threads; sub.temp_node.template_param = t; break; }
        case SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE: { auto *t = new shared_memory_total_warp_reduce_template_node_param_t(); t->tblock_num = tblock; t->thread_num_in_block = threads; t->thread_num_of_row_reduce = row_reduce; sub.temp_node.template_param = t; break; }
        case DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE: { auto *t = new direct_atom_total_warp_reduce_template_node_param_t(); t->tblock_num = tblock; t->thread_num_in_block = threads; sub.temp_node.template_param = t; break; }
        case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE: { auto *t = new unaligned_warp_reduce_same_TLB_size_template_node_param_t(); t->tblock_num = tblock; t->thread_num_in_block = threads; sub.temp_node.template_param = t; break; }
        case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE: { auto *t = new unaligned_warp_reduce_same_TLB_size_template_with_warp_reduce_node_param_t(); t->thread_num_in_block = threads; sub.temp_node.template_param = t; break; }
        default: return -1;
      }
      graph.compressed_sub_block_exe_graph_and_template_vec.push_back(sub);
    }
    if (at != n_desc) return -1;
    text = convert_dense_view_matrix_and_compressed_sub_block_exe_graph_and_template_to_string_safety(graph);
  }
  if (with_frame) {
    std::ostringstream f;
    f << "gflops:" << gflops << std::endl;
    f << "time:" << time_ms << std::endl;
    if (gflops != 0) f << text << std::endl; else f << "error" << std::endl;
    f << "finish search" << std::endl;
    text = f.str();
  }
  return put_text(text, out, cap);
}

}  // extern "C"
