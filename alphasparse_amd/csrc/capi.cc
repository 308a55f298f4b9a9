// extern "C" surface declared in include/alphasparse_amd.h (matrix / graph part).
#include "capi_internal.hpp"
#include "device_facts.hpp"

#include <cstring>

thread_local std::string g_as_last_error;

extern "C" {

const char *as_last_error(void) { return g_as_last_error.c_str(); }
const char *as_version(void) { return "alphasparse_amd 0.1 (gfx950)"; }

int as_device_facts(uint64_t *cu_num, uint64_t *lds_bytes, uint64_t *xcd_num, uint64_t *l2_bytes_per_xcd, int *from_device) {
  AS_API_BEGIN
  const asx::DeviceFacts &f = asx::device_facts();
  if (cu_num) *cu_num = f.cu_num;
  if (lds_bytes) *lds_bytes = f.lds_bytes;
  if (xcd_num) *xcd_num = asx::kXcdNum;
  if (l2_bytes_per_xcd) *l2_bytes_per_xcd = asx::kL2BytesPerXcd;
  if (from_device) *from_device = f.from_device ? 1 : 0;
  return 0;
  AS_API_END(-1)
}

int as_device_facts_read(int device) {
  AS_API_BEGIN
  asx::read_device_facts(device);
  return 0;
  AS_API_END(-1)
}

int as_device_facts_reset(void) {
  AS_API_BEGIN
  asx::reset_device_facts();
  return 0;
  AS_API_END(-1)
}

int as_device_facts_set(uint64_t cu_num, uint64_t lds_bytes) {
  AS_API_BEGIN
  AS_CHECK(lds_bytes == 0 || lds_bytes >= 65536, "at least 64 KB of LDS per workgroup");
  asx::set_device_facts(cu_num, lds_bytes);
  return 0;
  AS_API_END(-1)
}

as_matrix *as_matrix_from_coo(uint64_t rows, uint64_t cols, uint64_t nnz, const uint64_t *row, const uint64_t *col,
                              const double *val, int val_dtype, int wave) {
  AS_API_BEGIN
  AS_CHECK(row && col && val && nnz > 0, "null or empty COO input");
  AS_CHECK(rows > 0 && cols > 0, "empty matrix");
  asx::CooInput in;
  in.row.assign(row, row + nnz);
  in.col.assign(col, col + nnz);
  in.val.assign(val, val + nnz);
  in.row_index_max = rows - 1;
  in.col_index_max = cols - 1;
  in.val_dtype = (asx::DType)val_dtype;
  for (uint64_t i = 0; i < nnz; i++) AS_CHECK(row[i] < rows && col[i] < cols, "index out of the matrix");
  auto *h = new as_matrix();
  h->m = asx::matrix_from_coo(in, (unsigned)wave);
  return h;
  AS_API_END(nullptr)
}

as_matrix *as_matrix_from_coo_file(const char *path, int val_dtype, int wave) {
  AS_API_BEGIN
  AS_CHECK(path, "null path");
  asx::CooInput in = asx::read_coo_file(path, (asx::DType)val_dtype);
  AS_CHECK(!in.row.empty(), "file holds no element");
  auto *h = new as_matrix();
  h->m = asx::matrix_from_coo(in, (unsigned)wave);
  return h;
  AS_API_END(nullptr)
}

as_matrix *as_matrix_from_mtx_file(const char *path, int val_dtype, int wave, int keep_values) {
  AS_API_BEGIN
  AS_CHECK(path, "null path");
  asx::CooInput in = asx::read_mtx_file(path, (asx::DType)val_dtype, keep_values != 0);
  auto *h = new as_matrix();
  h->m = asx::matrix_from_coo(in, (unsigned)wave);
  return h;
  AS_API_END(nullptr)
}

as_matrix *as_matrix_from_binary_file(const char *path, int wave) {
  AS_API_BEGIN
  AS_CHECK(path, "null path");
  asx::CooInput in = asx::read_coo_binary(path);
  auto *h = new as_matrix();
  h->m = asx::matrix_from_coo(in, (unsigned)wave);
  return h;
  AS_API_END(nullptr)
}

as_matrix *as_matrix_clone(const as_matrix *m) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  auto *h = new as_matrix();
  h->m = m->m->clone();
  return h;
  AS_API_END(nullptr)
}

void as_matrix_free(as_matrix *m) { delete m; }

static asx::CooInput coo_view(const asx::Matrix &m) {
  asx::CooInput in;
  in.row = m.coo_row; in.col = m.coo_col; in.val = m.coo_val;
  in.row_index_max = m.rows - 1; in.col_index_max = m.cols - 1; in.val_dtype = m.val_dtype;
  return in;
}

int as_matrix_check_sorted(const as_matrix *m) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  return asx::check_coo_sorted(coo_view(*m->m)) ? 1 : 0;
  AS_API_END(-1)
}

int as_matrix_has_empty_row(const as_matrix *m) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  return asx::coo_has_empty_row(coo_view(*m->m)) ? 1 : 0;
  AS_API_END(-1)
}

int64_t as_matrix_long_short_row_decomposition(const as_matrix *m, const uint64_t *low_bounds, uint64_t n_bounds,
                                               as_matrix **parts, uint64_t cap) {
  AS_API_BEGIN
  AS_CHECK(m && m->m && low_bounds && parts, "null argument");
  auto out = asx::long_short_row_decomposition(*m->m, std::vector<uint64_t>(low_bounds, low_bounds + n_bounds));
  AS_CHECK(out.size() <= cap, "more parts than the caller has room for");
  for (size_t i = 0; i < out.size(); i++) parts[i] = new as_matrix{std::move(out[i])};
  return (int64_t)out.size();
  AS_API_END(-1)
}

int as_matrix_total_row_level_padding(as_matrix *m, uint64_t multiple, int position, uint64_t input_col_index) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  asx::total_row_level_padding(*m->m, multiple, (asx::PaddingPosition)position, input_col_index);
  return 0;
  AS_API_END(-1)
}

int as_matrix_total_row_level_padding_direct(as_matrix *m, uint64_t target_size, unsigned padding_col_num,
                                             int position, uint64_t input_col_index) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  asx::total_row_level_padding_direct(*m->m, target_size, padding_col_num, (asx::PaddingPosition)position,
                                      input_col_index);
  return 0;
  AS_API_END(-1)
}

int as_matrix_total_row_level_padding_add(as_matrix *m, uint64_t add_size, unsigned padding_col_num, int position,
                                          uint64_t input_col_index) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  asx::total_row_level_padding_add(*m->m, add_size, padding_col_num, (asx::PaddingPosition)position, input_col_index);
  return 0;
  AS_API_END(-1)
}

int as_matrix_dense_col_level_padding(as_matrix *m, const uint64_t *row_index, const uint64_t *padding_target_size,
                                      uint64_t n) {
  AS_API_BEGIN
  AS_CHECK(m && m->m && (n == 0 || (row_index && padding_target_size)), "null argument");
  asx::dense_col_level_padding(*m->m, std::vector<uint64_t>(row_index, row_index + n),
                               std::vector<uint64_t>(padding_target_size, padding_target_size + n));
  return 0;
  AS_API_END(-1)
}

int as_matrix_remove_empty_rows(as_matrix *m) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  asx::remove_empty_rows(*m->m);
  return 0;
  AS_API_END(-1)
}

int64_t as_matrix_y_rows(const as_matrix *m) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  return (int64_t)m->m->y_rows;
  AS_API_END(-1)
}

int as_matrix_info(const as_matrix *m, uint64_t out[8]) {
  AS_API_BEGIN
  AS_CHECK(m && m->m && out, "null argument");
  const asx::Matrix &x = *m->m;
  out[0] = x.rows; out[1] = x.cols; out[2] = x.nnz; out[3] = x.origin_nnz; out[4] = x.items.size();
  out[5] = x.is_sorted; out[6] = x.is_compressed; out[7] = x.wave;
  return 0;
  AS_API_END(-1)
}

int as_matrix_set_option(as_matrix *m, const char *key, long value) {
  AS_API_BEGIN
  AS_CHECK(m && m->m && key, "null argument");
  if (!strcmp(key, "val_copy_from_zero_quirk")) m->m->val_copy_from_zero_quirk = value != 0;
  else throw asx::Error(std::string("unknown option ") + key);
  return 0;
  AS_API_END(-1)
}

int as_matrix_write_coo_file(const as_matrix *m, const char *path) {
  AS_API_BEGIN
  AS_CHECK(m && m->m && path, "null argument");
  const asx::Matrix &x = *m->m;
  asx::write_coo_file(path, x.rows, x.cols, x.coo_row, x.coo_col, x.coo_val, x.val_dtype);
  return 0;
  AS_API_END(-1)
}

int as_matrix_write_binary_file(const as_matrix *m, const char *path) {
  AS_API_BEGIN
  AS_CHECK(m && m->m && path, "null argument");
  const asx::Matrix &x = *m->m;
  AS_CHECK(!x.coo_row.empty(), "the matrix no longer holds its COO arrays");
  asx::CooInput in;
  in.row = x.coo_row;
  in.col = x.coo_col;
  in.val = x.coo_val;
  in.row_index_max = x.rows - 1;
  in.col_index_max = x.cols - 1;
  in.val_dtype = x.val_dtype;
  asx::write_coo_binary(path, in);
  return 0;
  AS_API_END(-1)
}

int as_execute_node(as_matrix *m, int node_type, int64_t sub, const long *scalars, int n_scalars, const uint64_t *list,
                    uint64_t n_list, const uint64_t *counts, uint64_t n_counts) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  AS_CHECK((n_scalars == 0 || scalars) && (n_list == 0 || list) && (n_counts == 0 || counts), "null parameter array");
  asx::ExeNode n;
  n.type = (asx::ExeNodeType)node_type;
  auto nested = [&]() {
    uint64_t k = 0;
    for (uint64_t i = 0; i < n_counts; i++) {
      AS_CHECK(k + counts[i] <= n_list, "counts exceed the list length");
      std::vector<uint32_t> v(counts[i]);
      for (uint64_t j = 0; j < counts[i]; j++) v[j] = (uint32_t)list[k + j];
      n.nested_block_size.push_back(std::move(v));
      k += counts[i];
    }
    AS_CHECK(k == n_list, "counts do not cover the list");
  };
  switch (n.type) {
    case asx::COMPRESSED_ROW_PADDING:
      AS_CHECK(n_scalars == 2, "need {multiply, padding_row_length}");
      n.multiply = scalars[0];
      n.padding_row_length = scalars[1];
      break;
    case asx::COMPRESSED_THREAD_LEVEL_NNZ_DIV:
      AS_CHECK(n_scalars == 1, "need {TLB_nnz_num}");
      n.TLB_nnz_num = scalars[0];
      break;
    case asx::COMPRESSED_THREAD_LEVEL_COL_DIV:
      n.col_num_of_TLB_in_each_parent_block.assign(list, list + n_list);
      break;
    case asx::COMPRESSED_TBLOCK_LEVEL_ROW_DIV:
      for (uint64_t i = 0; i < n_list; i++) n.row_num_of_each_BLB.push_back((uint32_t)list[i]);
      break;
    case asx::COMPRESSED_TBLOCK_LEVEL_COL_DIV:
    case asx::COMPRESSED_WARP_LEVEL_ROW_DIV:
    case asx::COMPRESSED_WARP_LEVEL_COL_DIV:
      nested();
      break;
    case asx::DENSE_ROW_COARSE_SORT:
      n.bin_row_nnz_low_bound.assign(list, list + n_list);
      break;
    case asx::DENSE_ROW_DIV:  // scalars (optional): {dense_sub_block_id [, height of equal strips when the list is empty]}
      n.row_div_position.assign(list, list + n_list);
      if (n_scalars >= 1) n.dense_sub_block_id = (uint64_t)scalars[0];
      if (n_scalars >= 2) n.fixed_row_block_size = scalars[1];
      break;
    case asx::DENSE_FINE_SORT:
      n.first_row_of_each_sort_band.assign(list, list + n_list);
      break;
    case asx::COMPRESSED_BLOCK_SORT:
      n.sort_block_index_arr.assign(list, list + n_list);
      break;
    case asx::DENSE_FIXED_COL_DIV:
      AS_CHECK(n_scalars >= 1, "need {fixed_col_block_size [, dense_sub_block_id]}");
      n.fixed_col_block_size = scalars[0];
      if (n_scalars >= 2) n.dense_sub_block_id = (uint64_t)scalars[1];
      break;
    default:
      break;
  }
  if (sub < 0) asx::execute_dense_node(*m->m, n);
  else asx::execute_exe_node_in_compressed_sub_matrix(*m->m, (uint64_t)sub, n);
  return 0;
  AS_API_END(-1)
}

int as_execute_strategy(as_matrix *m, int strategy, int64_t sub, const long p[4]) {
  AS_API_BEGIN
  AS_CHECK(m && m->m && p, "null argument");
  asx::StrategyNode n = asx::make_strategy((asx::ParamStrategy)strategy, p[0], p[1], p[2], p[3]);
  if (sub < 0) {
    asx::execute_param_strategy_node_of_dense_matrix(n, *m->m);
    asx::execute_dense_node(*m->m, n.node);
  } else {
    asx::execute_param_strategy_node_of_sub_compressed_matrix(n, *m->m, (uint64_t)sub);
    asx::execute_exe_node_in_compressed_sub_matrix(*m->m, (uint64_t)sub, n.node);
  }
  return 0;
  AS_API_END(-1)
}

int as_complete_blocking(as_matrix *m, int64_t sub) {
  AS_API_BEGIN
  AS_CHECK(m && m->m && sub >= 0, "bad argument");
  asx::execute_default_div_to_complete_each_level_blocking(*m->m, (uint64_t)sub);
  return 0;
  AS_API_END(-1)
}

static int64_t put_u64(const std::vector<uint64_t> &v, asx::DType dt, uint64_t *out, uint64_t cap, int *dtype) {
  if (dtype) *dtype = (int)dt;
  if (out) memcpy(out, v.data(), sizeof(uint64_t) * std::min<uint64_t>(cap, v.size()));
  return (int64_t)v.size();
}

int64_t as_matrix_get_u64(const as_matrix *m, int64_t sub, int slot, int field, uint64_t *out, uint64_t cap, int *dtype) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  const asx::Matrix &x = *m->m;
  if (slot == AS_SLOT_SORTED_ROW_INDEX) {
    if (!x.sorted_row_index.present) return -1;
    return put_u64(x.sorted_row_index.v, x.sorted_row_index.dt, out, cap, dtype);
  }
  if (slot == AS_SLOT_COO) return put_u64(field == 0 ? x.coo_row : x.coo_col, asx::UNSIGNED_LONG, out, cap, dtype);
  AS_CHECK(sub >= 0 && (uint64_t)sub < x.items.size(), "sub-matrix id out of range");
  const asx::DenseItem &it = x.items[sub];
  if (slot == AS_SLOT_DENSE_ITEM) {
    std::vector<uint64_t> v{it.min_row, it.max_row, it.min_col, it.max_col, it.begin_coo, it.end_coo, it.is_col_blocked};
    return put_u64(v, asx::UNSIGNED_LONG, out, cap, dtype);
  }
  AS_CHECK(it.cb != nullptr, "sub-matrix is not compressed");
  const asx::CompressedBlock &cb = *it.cb;
  if (slot == AS_SLOT_Y_WRITE_INDEX) {
    if (!cb.y_write_index.present) return -1;
    return put_u64(cb.y_write_index.v, cb.y_write_index.dt, out, cap, dtype);
  }
  if (slot == AS_SLOT_SHARE_FLAGS) {
    std::vector<uint64_t> v{cb.share_row_with_other_block, cb.share_row_with_other_warp, cb.share_row_with_other_thread,
                            cb.read_index.size()};
    return put_u64(v, asx::UNSIGNED_LONG, out, cap, dtype);
  }
  AS_CHECK(slot >= 0 && slot < 7, "bad slot");
  if ((size_t)slot >= cb.read_index.size()) return -1;
  const asx::Index &ix = *cb.read_index[slot];
  if (field == AS_F_SCALARS) {
    std::vector<uint64_t> v{ix.block_num, ix.length, ix.max_row, ix.min_row, ix.max_col, ix.min_col,
                            (uint64_t)ix.level, (uint64_t)ix.ctype, (uint64_t)ix.itype};
    return put_u64(v, asx::UNSIGNED_LONG, out, cap, dtype);
  }
  const asx::IArr *a = nullptr;
  switch (field) {
    case AS_F_INDEX_ARR: a = &ix.index_arr; break;
    case AS_F_FIRST_ROW: a = &ix.first_row; break;
    case AS_F_ROW_NUMBER: a = &ix.row_number; break;
    case AS_F_COO_BEGIN: a = &ix.coo_begin; break;
    case AS_F_COO_BLOCK_SIZE: a = &ix.coo_block_size; break;
    default: throw asx::Error("bad field");
  }
  if (!a->present) return -1;
  return put_u64(a->v, a->dt, out, cap, dtype);
  AS_API_END(-2)
}

int64_t as_matrix_get_f64(const as_matrix *m, int64_t sub, int which, double *out, uint64_t cap) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  const asx::Matrix &x = *m->m;
  const asx::ValVec *v = nullptr;
  if (which == AS_V_COO_VALUE_CACHE) v = &x.coo_val;
  else {
    AS_CHECK(sub >= 0 && (uint64_t)sub < x.items.size() && x.items[sub].cb, "sub-matrix is not compressed");
    const asx::CompressedBlock &cb = *x.items[sub].cb;
    const asx::ValPtr &p = which == AS_V_VAL ? cb.val : which == AS_V_PADDING_VAL ? cb.padding_val : cb.staggered_val;
    if (!p) return -1;
    v = p.get();
  }
  if (out) memcpy(out, v->data(), sizeof(double) * std::min<uint64_t>(cap, v->size()));
  return (int64_t)v->size();
  AS_API_END(-2)
}

}  // extern "C"
