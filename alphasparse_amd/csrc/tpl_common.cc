// Helpers shared by the kernel-template families.
#include "templates.hpp"

namespace asx {

const char *convert_template_type_to_string(TemplateType t) {
  static const char *n[] = {"DIRECT_ATOM_TEMPLATE", "DIRECT_ATOM_TEMPLATE_WARP_COMPRESS",
                            "DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS", "SHARED_MEMORY_TEMPLATE",
                            "SHARED_MEMORY_TEMPLATE_WARP_COMPRESS", "SHARED_MEMORY_LONG_ROW_TEMPLATE",
                            "SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE", "DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE",
                            "UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE",
                            "UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE", "EMPTY_TEMPLATE",
                            "NONE_TEMPLATE", "SHARED_MEMORY_X_SLICE_TEMPLATE", "SHARED_MEMORY_TILE_TEMPLATE",
                            "SHARED_MEMORY_PRODUCT_BIN_TEMPLATE"};
  AS_CHECK(t >= 0 && t < TEMPLATE_TYPE_COUNT, "unknown template type");
  return n[(int)t];
}

uint64_t template_format_bytes(const Template &t) {
  uint64_t b = t.val_arr.size() * (uint64_t)dtype_size(t.val_dtype) +
               t.col_index_arr.size() * (uint64_t)dtype_size(t.col_index_arr.dt);
  for (auto &a : t.arrays)
    if (a.passed()) b += a.a.size() * (uint64_t)dtype_size(a.a.dt);
  b += 2 * t.scratch_bytes;  // accumulated into, then read back and cleared
  return b;
}

std::vector<uint64_t> global_row_of_each_TLB(const CompressedBlock &cb) {
  AS_CHECK(cb.read_index.size() == 7, "blocking is incomplete");
  const Index &bl = *cb.read_index[2], &wl = *cb.read_index[3], &tl = *cb.read_index[4];
  AS_CHECK(!tl.row_number.present, "row num in thread level block must be 1");
  std::vector<uint64_t> row(tl.block_num);
  for (uint64_t b = 0; b < bl.block_num; b++)
    for (uint64_t w = bl.index_arr[b]; w < bl.index_arr[b + 1]; w++)
      for (uint64_t t = wl.index_arr[w]; t < wl.index_arr[w + 1]; t++) {
        AS_CHECK(t < tl.block_num, "TLB offset beyond the TLB level");
        row[t] = bl.first_row[b] + wl.first_row[w] + tl.first_row[t];
      }
  return row;
}

bool sub_block_is_col_restricted(const Matrix &m, uint64_t sub) {
  const DenseItem &it = m.items[sub];
  return !(it.min_col == 0 && it.max_col == m.cols - 1);
}

uint64_t effective_unit_num(const Matrix &m, uint64_t sub, const std::vector<uint64_t> &unit_row) {
  const DenseItem &it = m.items[sub];
  const Index &ri = *it.cb->read_index[0];
  if (it.max_row >= ri.max_row) return unit_row.size();
  uint64_t dense_rows = it.max_row - it.min_row + 1;
  for (uint64_t u = 0; u < unit_row.size(); u++)
    if (unit_row[u] >= dense_rows) {
      for (uint64_t v = u; v < unit_row.size(); v++)
        AS_CHECK(unit_row[v] >= dense_rows, "padding rows must be the last rows of the sub-matrix");
      return u;
    }
  throw Error("effective_unit_num: row padding left no padded unit");
}

bool apply_global_sort(const Matrix &m, uint64_t sub, std::vector<uint64_t> &unit_row, uint64_t effective) {
  const CompressedBlock &cb = *m.items[sub].cb;
  if (cb.y_write_index.present) {
    // rows sorted inside BLBs: back to the rows of the sub-matrix; they stay relative to its first row, and a
    // sort of the whole matrix (or the map of remove_empty_rows) may follow below
    for (uint64_t u = 0; u < effective; u++) {
      AS_CHECK(unit_row[u] < cb.y_write_index.size(), "row outside the permutation of the BLB sort");
      unit_row[u] = cb.y_write_index[unit_row[u]];
    }
  }
  if (!m.sorted_row_index.present) return false;
  uint64_t first = m.items[sub].min_row;
  for (uint64_t u = 0; u < effective; u++) {
    uint64_t r = unit_row[u] + first;
    AS_CHECK(r < m.sorted_row_index.size(), "row outside the sort permutation");
    unit_row[u] = m.sorted_row_index[r];
  }
  return true;
}

void init_template_common(Template &t, TemplateType type, const Matrix &m, uint64_t sub) {
  AS_CHECK(sub < m.items.size() && m.items[sub].cb, "sub-matrix is not compressed");
  t.type = type;
  t.sub = sub;
  t.wave = m.wave;
  t.val_dtype = m.val_dtype;
  t.matrix_rows = m.rows;
  t.matrix_cols = m.cols;
  t.kernal_first_row_index = m.items[sub].min_row;
  t.kernal_first_col_index = m.items[sub].min_col;
  t.origin_nnz = m.items[sub].end_coo - m.items[sub].begin_coo + 1;
  t.local_sort_index = m.items[sub].cb->y_write_index.present;
  const CompressedBlock &cb = *m.items[sub].cb;
  t.padding_arr_size = cb.padding_val ? cb.padding_val->size() : (cb.val ? cb.val->size() : 0);
}

bool template_needs_cleared_y(const Template &t, const Matrix &m, uint64_t sub) {
  if (t.is_atom_add) return true;
  if (t.type == EMPTY_TEMPLATE) return true;  // no kernel: the clear is what writes the rows of this sub-matrix
  // the CSR5-like pair adds the partial sums of rows that cross a tile or a wavefront into y
  if (t.type == UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE ||
      t.type == UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE)
    return true;
  // the two-kernel LDS templates store every row of the strip in their finish kernel, with or without elements
  if (t.finish_tblock_num && (t.type == SHARED_MEMORY_TILE_TEMPLATE || t.type == SHARED_MEMORY_PRODUCT_BIN_TEMPLATE))
    return false;
  // the tile template under row ownership stores every row of every row group that holds an element, zeros
  // included; a row group without any element has no run and is stored by nobody
  if (t.type == SHARED_MEMORY_TILE_TEMPLATE && t.own_rows) return t.sc("row_groups_without_elements") != 0;
  // the row-wise templates store the rows that have a unit (TLB, WLB or BLB): a row without elements has none
  const DenseItem &it = m.items[sub];
  const uint64_t sub_rows = it.max_row - it.min_row + 1;
  std::vector<bool> seen(sub_rows, false);
  uint64_t count = 0;
  for (uint64_t r : it.cb->read_index[0]->index_arr.v)
    if (r < sub_rows && !seen[r]) {
      seen[r] = true;
      count++;
    }
  return count != sub_rows;
}

#define AS_DISPATCH(type, call)                                                                         \
  switch (type) {                                                                                       \
    case DIRECT_ATOM_TEMPLATE: return tpl_direct_atom::call;                                            \
    case DIRECT_ATOM_TEMPLATE_WARP_COMPRESS: return tpl_direct_atom_warp_compress::call;                \
    case DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS: return tpl_direct_atom_warp_block_compress::call;    \
    case SHARED_MEMORY_TEMPLATE: return tpl_shared_memory::call;                                        \
    case SHARED_MEMORY_TEMPLATE_WARP_COMPRESS: return tpl_shared_memory_warp_compress::call;            \
    case SHARED_MEMORY_LONG_ROW_TEMPLATE: return tpl_shared_memory_long_row::call;                      \
    case SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE: return tpl_shared_memory_total_warp_reduce::call;    \
    case DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE: return tpl_direct_atom_total_warp_reduce::call;        \
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE: return tpl_unaligned_warp_reduce::call;          \
    case UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE:                                 \
      return tpl_unaligned_warp_reduce_with_warp_reduce::call;                                          \
    case EMPTY_TEMPLATE: return tpl_empty::call;                                                        \
    case SHARED_MEMORY_X_SLICE_TEMPLATE: return tpl_shared_memory_x_slice::call;                        \
    case SHARED_MEMORY_TILE_TEMPLATE: return tpl_shared_memory_tile::call;                              \
    case SHARED_MEMORY_PRODUCT_BIN_TEMPLATE: return tpl_shared_memory_product_bin::call;                \
    default: throw Error(std::string("template type is not supported: ") + convert_template_type_to_string(type)); \
  }

bool is_supported_by_template(TemplateType type, const Matrix &m, uint64_t sub) {
  AS_CHECK(sub < m.items.size() && m.items[sub].cb && m.items[sub].cb->read_index.size() == 7,
           "blocking of the sub-matrix is incomplete");
  // a tile-ordered sub-matrix (elements no longer sorted by row) is readable by its own template only
  if ((m.items[sub].cb->row_group != 0) != (type == SHARED_MEMORY_TILE_TEMPLATE || type == SHARED_MEMORY_PRODUCT_BIN_TEMPLATE))
    return false;
  AS_DISPATCH(type, is_supported(m, sub))
}
std::unique_ptr<Template> init_template(TemplateType type, const Matrix &m, uint64_t sub) {
  AS_CHECK(sub < m.items.size() && m.items[sub].cb && m.items[sub].cb->read_index.size() == 7,
           "blocking of the sub-matrix is incomplete");
  AS_DISPATCH(type, init(m, sub))
}
void try_all_compress(Template &t) { AS_DISPATCH(t.type, try_all_compress(t)) }
void set_default_launch(Template &t) { AS_DISPATCH(t.type, set_default_launch(t)) }
namespace tpl_direct_atom_warp_block_compress { bool make_columns_relative(Template &t); bool make_columns_diagonal(Template &t); }
bool make_columns_diagonal(Template &t) {
  return t.type == DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS && tpl_direct_atom_warp_block_compress::make_columns_diagonal(t);
}
bool make_columns_relative(Template &t) {
  return t.type == DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS && tpl_direct_atom_warp_block_compress::make_columns_relative(t);
}
namespace tpl_shared_memory_tile { std::unique_ptr<Template> init_with_column_runs(const Matrix &m, uint64_t sub); }
std::unique_ptr<Template> init_tile_template_with_column_runs(const Matrix &m, uint64_t sub) {
  AS_CHECK(is_supported_by_template(SHARED_MEMORY_TILE_TEMPLATE, m, sub), "format is not supported by SHARED_MEMORY_TILE_TEMPLATE");
  return tpl_shared_memory_tile::init_with_column_runs(m, sub);
}
namespace tpl_shared_memory_tile { std::unique_ptr<Template> init_variant(const Matrix &m, uint64_t sub, bool column_runs, bool own_rows, uint64_t row_block); }
namespace tpl_shared_memory_tile { uint64_t row_block_guess(const Matrix &m, uint64_t sub); }
uint64_t tile_row_block_guess(const Matrix &m, uint64_t sub) { return tpl_shared_memory_tile::row_block_guess(m, sub); }
namespace tpl_shared_memory_tile { uint64_t column_run_stream_estimate(const Matrix &m, uint64_t sub); }
uint64_t tile_column_run_stream_estimate(const Matrix &m, uint64_t sub) {
  return tpl_shared_memory_tile::column_run_stream_estimate(m, sub);
}

std::unique_ptr<Template> init_tile_template_variant(const Matrix &m, uint64_t sub, bool column_runs, bool own_rows, uint64_t row_block) {
  AS_CHECK(is_supported_by_template(SHARED_MEMORY_TILE_TEMPLATE, m, sub), "format is not supported by SHARED_MEMORY_TILE_TEMPLATE");
  return tpl_shared_memory_tile::init_variant(m, sub, column_runs, own_rows, row_block);
}
std::string code_of_template_kernal(const Template &t) { AS_DISPATCH(t.type, kernel_source(t)) }

std::vector<std::string> kernel_array_args(const Template &t) {
  std::vector<std::string> v;
  for (auto &a : t.arrays)
    if (a.passed()) v.push_back(a.name);
  return v;
}

}  // namespace asx
