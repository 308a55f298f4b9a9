// Format operators (the upstream op_manager.hpp API, same names and argument
// meaning) over the typed data model.  Errors that upstream turns into
// assert(false) are thrown as asx::Error.
#pragma once
#include "as_types.hpp"

namespace asx {

// Dense-view operators ------------------------------------------------------
// No upstream counterpart (upstream stops at a matrix with rows that hold no element, main.cc:604-621):
// the rows that hold elements are renumbered 0, 1, 2, ... in their order, sorted_row_index[new] = old maps
// them back to y, whose other entries stay at the zero every SpMV clears them to.  Must come first.
void remove_empty_rows(Matrix &m);
// total_dense_block_coarse_sort (op_manager.cc:5492)
std::vector<uint64_t> total_dense_block_coarse_sort(Matrix &m, const std::vector<uint64_t> &bin_row_nnz_low_bound);
// long_short_row_decomposition (op_manager.cc:9-124): A = A_0 + A_1 + ..., one matrix per class of row
// length.  low_bounds[0] = 0 and ascending; a row of n elements goes to the last class whose bound is
// <= n.  Every part keeps the shape of A and the original row numbers (the rows of the other classes
// are empty in it), classes without rows are left out, and at least two parts must come out.
// Before any other operator.  Upstream frees the input; here it is left untouched.
std::vector<std::unique_ptr<Matrix>> long_short_row_decomposition(const Matrix &m, const std::vector<uint64_t> &low_bounds);
// total_dense_block_sort (op_manager.cc:4780; banded form :4871): rows by length, longest first, rows of equal
// length in their previous order (upstream sorts by insertion); with bands, inside every band of rows
// [first[i], first[i+1]) (the last band ends with the matrix).  sorted_row_index[new] = old.
// op_manager.cc:4104 compressed_block_sort: rows of the listed BLBs by falling length, permutation in y_write_index
void compressed_block_sort(CompressedBlock &cb, const std::vector<uint64_t> &sort_block_index_arr,
                           uint64_t real_rows = ~0ull);
void total_dense_block_sort(Matrix &m, const std::vector<uint64_t> &first_row_of_each_sort_band = {});
// global_padding_position (op_manager.hpp:13): where total_row_level_padding* puts the rows it adds
enum PaddingPosition { TOP_PADDING = 0, END_PADDING = 1 };
// total_row_level_padding (op_manager.cc:5361): rows up to the next multiple of `multiple` (nothing when it is
// one already), every added row with one zero; END: the rows follow the matrix, their zero in column
// input_col_index; TOP: they precede it (row r becomes row r + added), their zero in column 0.  y grows with the
// matrix.  Before any other operator.
void total_row_level_padding(Matrix &m, uint64_t multiple, PaddingPosition position = END_PADDING,
                             uint64_t input_col_index = 0);
// total_row_level_padding_direct (op_manager.cc:5221): rows up to target_size (> rows).  END: every added row
// holds padding_col_num zeros in columns input_col_index, input_col_index + 1, ...; TOP: one zero in column 0
// (upstream's TOP branch writes one element per row and then asserts the count, so only padding_col_num == 1
// passes there; the same is required here).
void total_row_level_padding_direct(Matrix &m, uint64_t target_size, unsigned padding_col_num = 1,
                                    PaddingPosition position = END_PADDING, uint64_t input_col_index = 0);
// total_row_level_padding_add (op_manager.hpp:221): add_size more rows
void total_row_level_padding_add(Matrix &m, uint64_t add_size, unsigned padding_col_num = 1,
                                 PaddingPosition position = END_PADDING, uint64_t input_col_index = 0);
// dense_col_level_padding (op_manager.cc:5043), whole-matrix form: row row_index[i] is filled with zeros up to
// padding_target_size[i] elements (more than it holds), each in the column of the row's last element (column 0
// in a row without elements).
void dense_col_level_padding(Matrix &m, const std::vector<uint64_t> &row_index,
                             const std::vector<uint64_t> &padding_target_size);
// var_len_row_div (op_manager.cc:370), sub_block == NULL form
void var_len_row_div(Matrix &m, const std::vector<uint64_t> &block_first_row_csr_index);
// fixed_len_row_div (op_manager.cc:127), whole-matrix form
void fixed_len_row_div(Matrix &m, uint64_t len);
// fixed_len_col_div (op_manager.cc:665), whole-matrix form: column bands of `len` columns, every band a
// sub-block over all rows (is_col_blocked), bands without elements dropped
void fixed_len_col_div(Matrix &m, uint64_t len);
// The three divisions applied to sub-block `sub` of an already divided matrix (op_manager.cc:243-365, 808-965;
// upstream's var_len_row_div stops with "further div is not support", :520): positions are relative to the
// sub-block's first row, bands are counted from its first column; the parent leaves the table, its parts are
// appended at the end.
void var_len_row_div(Matrix &m, const std::vector<uint64_t> &block_first_row_csr_index, uint64_t sub);
void fixed_len_row_div(Matrix &m, uint64_t len, uint64_t sub);
void fixed_len_col_div(Matrix &m, uint64_t len, uint64_t sub);
// compress_dense_view (op_manager.cc:968)
void compress_dense_view(Matrix &m);

// Compressed-view operators --------------------------------------------------
// compress_block_end_block_multiple_padding (op_manager.cc:5735)
void compress_block_end_block_multiple_padding(Matrix &m, uint64_t sub, uint64_t multiple, uint64_t padding_row_length);
// sep_tblock_level_row_csr (op_manager.cc:1270) and its two presets (:1525, :1540)
void sep_tblock_level_row_csr(CompressedBlock &cb, const std::vector<uint32_t> &block_size_arr);
void default_sep_tblock_level_row_csr(CompressedBlock &cb);
void one_row_sep_tblock_level_row_csr(CompressedBlock &cb);
// sep_tblock_level_col_csr (op_manager.cc:1566)
void sep_tblock_level_col_csr(CompressedBlock &cb, const std::vector<uint64_t> &block_index_arr,
                              const std::vector<std::vector<uint32_t>> &block_size_arr);
// sep_warp_level_row_csr (op_manager.cc:1970) and presets (:2361, :2376)
void sep_warp_level_row_csr(CompressedBlock &cb, const std::vector<uint64_t> &block_index_arr,
                            const std::vector<std::vector<uint32_t>> &row_block_size_arr);
void default_sep_warp_level_row_csr(CompressedBlock &cb);
void one_row_sep_warp_level_row_csr(CompressedBlock &cb);
// sep_warp_level_col_csr (op_manager.cc:2416); every WLB must be listed, as the
// graph node executor does (exe_graph.cc:1942-2041)
void sep_warp_level_col_csr(CompressedBlock &cb, const std::vector<uint64_t> &block_index_arr,
                            const std::vector<std::vector<uint32_t>> &col_block_size_arr);
// sep_thread_level_col_ell_with_padding (op_manager.cc:3105); `wave` replaces
// the literal 32 of the upstream code
void sep_thread_level_col_ell_with_padding(CompressedBlock &cb, const std::vector<uint64_t> &block_index_arr,
                                           const std::vector<uint64_t> &thread_col_block_size, unsigned wave);
// sep_thread_level_acc_to_nnz (op_manager.cc:3807)
void sep_thread_level_acc_to_nnz(CompressedBlock &cb, uint64_t thread_level_block_size);

// No upstream counterpart: 2-D BLBs.  Rows are cut into groups of `row_group` rows, columns into
// slices of `col_slice` columns; the elements are re-ordered by (slice, row group, row, column) and
// every (slice, row group) tile that holds elements becomes a run of BLBs of at most `block_nnz`
// elements.  Completes the blocking (one WLB per BLB, TLB size 1, no padding).
void sep_tblock_level_row_group_col_slice(CompressedBlock &cb, uint64_t col_slice, uint64_t row_group, uint64_t block_nnz);

// Row-length helpers (op_manager.cc:4360-4497)
std::vector<uint64_t> get_nnz_of_each_row_in_compressed_sub_matrix(const CompressedBlock &cb);
std::vector<uint64_t> get_nnz_of_each_row(const Matrix &m);

}  // namespace asx
