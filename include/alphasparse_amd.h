/*
 * alphasparse_amd -- C ABI of the MI355X SpMV format-and-kernel generator.
 *
 * The upstream project has no FFI layer: its boundary is a flat C++ API over POD
 * structs.  Each entry point below names the upstream function(s) it stands for
 * (paths relative to the upstream source tree).  All entry points use plain C
 * types, never abort the process, and report failures through a status code /
 * NULL plus as_last_error() (upstream: assert(false) / exit(-1)).
 *
 * Integer arrays are exchanged as uint64_t values together with the narrowed
 * element type (enum as_dtype) the format stores them in; the byte image of an
 * array is "values cast to that type".
 */
#ifndef ALPHASPARSE_AMD_H
#define ALPHASPARSE_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* struct.hpp:32-47 `enum data_type` (same ordinals) */
enum as_dtype {
  AS_CHAR, AS_UNSIGNED_CHAR, AS_SHORT, AS_UNSIGNED_SHORT, AS_INT, AS_UNSIGNED_INT, AS_LONG, AS_UNSIGNED_LONG,
  AS_LONG_LONG, AS_UNSIGNED_LONG_LONG, AS_FLOAT, AS_DOUBLE, AS_BOOL, AS_NONE_DATA_TYPE
};

/* exe_graph.hpp:36-57 `enum exe_node_type` (same ordinals) */
enum as_node_type {
  AS_BEGIN_INPUT_FILE, AS_BEGIN_ARTIFICIAL_INPUT, AS_BEGIN_MEMORY_CACHE_INPUT_FILE, AS_DENSE_ROW_COARSE_SORT,
  AS_DENSE_FINE_SORT, AS_DENSE_TOTAL_ROW_LEVEL_PADDING, AS_DENSE_BLOCK_SORT, AS_DENSE_ROW_DIV, AS_DENSE_FIXED_COL_DIV,
  AS_COMPRESS, AS_COMPRESSED_ROW_PADDING, AS_COMPRESSED_BLOCK_SORT, AS_COMPRESSED_THREAD_LEVEL_ROW_DIV,
  AS_COMPRESSED_THREAD_LEVEL_COL_DIV, AS_COMPRESSED_WARP_LEVEL_ROW_DIV, AS_COMPRESSED_WARP_LEVEL_COL_DIV,
  AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV, AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV, AS_COMPRESSED_THREAD_LEVEL_NNZ_DIV
};

/* parameter_set_strategy.hpp:7-22 `enum exe_node_param_set_strategy` (same ordinals) */
enum as_param_strategy {
  AS_COMPRESSED_ROW_PADDING_DIRECT, AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY,
  AS_COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ, AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED,
  AS_COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY, AS_COMPRESSED_WARP_LEVEL_COL_DIV_FIXED,
  AS_COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE, AS_COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED,
  AS_COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT, AS_DENSE_ROW_COARSE_SORT_FIXED,
  AS_DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT, AS_COMPRESS_NONE,
  AS_DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ,
  /* no counterpart in the reference (placed behind its ordinals): p[0] = column slice width; every row is cut
   * into BLBs where its columns cross a multiple of p[0], for kernels that keep one slice of x in LDS */
  AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE,
  /* no counterpart in the reference: p[0] = column slice width, p[1] = row group height, p[2] = BLB size; the
   * elements are re-ordered into 2-D tiles (row group x column slice) and every tile is cut into BLBs of at
   * most p[2] elements, for kernels that keep the slice of x and the row group's sums in LDS */
  AS_COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE
};

/* code_builder.hpp:15-29 `enum template_type` (same ordinals) */
enum as_template_type {
  AS_DIRECT_ATOM_TEMPLATE, AS_DIRECT_ATOM_TEMPLATE_WARP_COMPRESS, AS_DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS,
  AS_SHARED_MEMORY_TEMPLATE, AS_SHARED_MEMORY_TEMPLATE_WARP_COMPRESS, AS_SHARED_MEMORY_LONG_ROW_TEMPLATE,
  AS_SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE, AS_DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE,
  AS_UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE, AS_UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE,
  AS_EMPTY_TEMPLATE, AS_NONE_TEMPLATE,
  /* no counterpart in the reference (placed behind its ordinals): one-row BLBs cut at column slice boundaries,
   * the slice of x copied into LDS once per workgroup trip; for long rows with columns spread over a vector
   * larger than L2 */
  AS_SHARED_MEMORY_X_SLICE_TEMPLATE,
  /* no counterpart in the reference: 2-D tiles (row group x column slice) stored tile by tile; the slice of x
   * and the partial sums of the row group live in LDS, rows of any length, columns spread over a vector
   * larger than L2 */
  AS_SHARED_MEMORY_TILE_TEMPLATE,
  /* no counterpart in the reference: the same 2-D tiles in two passes; spmv_<sub> multiplies every element by
   * its x value from an LDS-resident slice and streams the products to scratch, spmv_<sub>_finish adds the
   * products of a row group up in LDS and stores the rows; short rows, columns spread over a vector larger
   * than L2, no gather from HBM */
  AS_SHARED_MEMORY_PRODUCT_BIN_TEMPLATE
};

/* Addressing of the arrays of one compressed sub-matrix (as_matrix_get_u64):
 * slot 0..6 = read_index[slot] (struct.hpp:60-118), field = one of as_index_field. */
enum as_index_field {
  AS_F_INDEX_ARR, AS_F_FIRST_ROW, AS_F_ROW_NUMBER, AS_F_COO_BEGIN, AS_F_COO_BLOCK_SIZE,
  /* scalars of the level: {block_num, length, max_row, min_row, max_col, min_col, level, compressed type, index type} */
  AS_F_SCALARS
};
enum as_special_slot {
  AS_SLOT_SORTED_ROW_INDEX = 100, /* sparse_struct_t::sorted_row_index (sub ignored) */
  AS_SLOT_DENSE_ITEM = 101,       /* {min_row,max_row,min_col,max_col,begin_coo,end_coo,is_col_blocked} */
  AS_SLOT_SHARE_FLAGS = 102,      /* {share_row_with_other_block, _warp, _thread, read_index.size()} */
  AS_SLOT_COO = 103,              /* field 0/1 = coo_row_index_cache / coo_col_index_cache (sub ignored) */
  AS_SLOT_Y_WRITE_INDEX = 104     /* compressed_block_t::y_write_index[0] (struct.hpp): the permutation of
                                   * compressed_block_sort, absent (-1) without it */
};
enum as_value_array { AS_V_VAL, AS_V_PADDING_VAL, AS_V_STAGGERED_PADDING_VAL, AS_V_COO_VALUE_CACHE };

typedef struct as_matrix as_matrix;     /* sparse_struct_t + operator_manager_t */
typedef struct as_builder as_builder;   /* code_builder_t: one kernel template per sub-matrix + device state */

/* Message of the last failure on the calling thread ("" if none). */
const char *as_last_error(void);
/* Library version string. */
const char *as_version(void);

/* ---- input: struct.cc:92-175 get_matrix_index_and_val_from_file,
 *      struct.cc:296-390 init_sparse_struct_by_coo_vector,
 *      exe_graph.cc:125 get_exe_begin_memory_cache_input_file_param_from_coo_file.
 * `wave` = lane count the thread-level operators pad and interleave for
 * (64 = CDNA wavefront; 32 reproduces the upstream arrays bit for bit).
 * `val` is always passed as double; val_dtype AS_FLOAT rounds every value to float. */
as_matrix *as_matrix_from_coo(uint64_t rows, uint64_t cols, uint64_t nnz, const uint64_t *row, const uint64_t *col,
                              const double *val, int val_dtype, int wave);
as_matrix *as_matrix_from_coo_file(const char *path, int val_dtype, int wave);
/* data_prepare.py:34-66 in one step: a Matrix Market coordinate file (.mtx) -> COO sorted by (row, column).
 * keep_values = 0 forces every value to 1 as the reference's script does; 1 keeps the file's values.  Beyond
 * the script: the banner is honoured (symmetric / hermitian / skew-symmetric entries are mirrored, pattern
 * entries get 1).  Empty rows are reported by as_matrix_has_empty_row, as for any other input. */
as_matrix *as_matrix_from_mtx_file(const char *path, int val_dtype, int wave, int keep_values);
/* binary cache of the COO input (no counterpart in the reference, whose struct.cc:92-175 parses text every
 * run): 64-byte header + row / column (u32 or u64) + value arrays */
as_matrix *as_matrix_from_binary_file(const char *path, int wave);
/* struct.cc:392 val_copy_from_old_matrix_struct */
as_matrix *as_matrix_clone(const as_matrix *m);
void as_matrix_free(as_matrix *m);
/* exe_graph.cc:3850 check_begin_memory_cache_input_file -> 1 sorted / 0 not;
 * exe_graph.cc:3916 has_empty_line_in_begin_memory_cache_input_file -> 1 has empty row / 0 none; <0 error */
int as_matrix_check_sorted(const as_matrix *m);
int as_matrix_has_empty_row(const as_matrix *m);
/* op_manager.cc:9 long_short_row_decomposition(matrix, row_nnz_low_bound_of_sub_matrix): A = sum of parts, one
 * per class of row length (low_bounds[0] = 0, ascending; a row of n elements goes to the last class whose bound
 * is <= n).  Every part has the shape of A and the original row numbers, classes without rows are left out, at
 * least two parts must come out.  Writes the new matrices (owned by the caller, as_matrix_free) to parts[0..)
 * and returns how many; -1 on error.  The reference frees its input; `m` is left untouched here.  A part has
 * rows without elements: as_matrix_remove_empty_rows is its next operator. */
int64_t as_matrix_long_short_row_decomposition(const as_matrix *m, const uint64_t *low_bounds, uint64_t n_bounds,
                                               as_matrix **parts, uint64_t cap);
/* op_manager.hpp:13 global_padding_position */
#define AS_TOP_PADDING 0
#define AS_END_PADDING 1
/* op_manager.cc:5361 total_row_level_padding(op_manager, multiple, padding_type, input_col_index): rows up to
 * the next multiple of `multiple` (no change when it is one), one zero per added row; AS_END_PADDING appends the
 * rows (zero in column input_col_index), AS_TOP_PADDING puts them first (zero in column 0, row r becomes row
 * r + added).  The matrix and y grow (as_matrix_info, as_matrix_y_rows).  Before any other operator. */
int as_matrix_total_row_level_padding(as_matrix *m, uint64_t multiple, int position, uint64_t input_col_index);
/* op_manager.cc:5221 total_row_level_padding_direct(op_manager, target_size, padding_col_num, padding_type,
 * input_col_index): rows up to target_size (> rows); AS_END_PADDING: padding_col_num zeros per added row in
 * columns input_col_index, input_col_index + 1, ...; AS_TOP_PADDING: padding_col_num must be 1 (the reference's
 * own element count only holds for 1), the zero sits in column 0. */
int as_matrix_total_row_level_padding_direct(as_matrix *m, uint64_t target_size, unsigned padding_col_num,
                                             int position, uint64_t input_col_index);
/* op_manager.hpp:221 total_row_level_padding_add: add_size more rows, otherwise as above */
int as_matrix_total_row_level_padding_add(as_matrix *m, uint64_t add_size, unsigned padding_col_num, int position,
                                          uint64_t input_col_index);
/* op_manager.cc:5043 dense_col_level_padding(op_manager, NULL, row_index_vec, padding_target_size_vec): row
 * row_index[i] is filled with zeros up to padding_target_size[i] elements (more than it holds), each in the
 * column of the row's last element (column 0 in a row without elements).  Before blocking. */
int as_matrix_dense_col_level_padding(as_matrix *m, const uint64_t *row_index, const uint64_t *padding_target_size,
                                      uint64_t n);
/* no counterpart in the reference (it stops at such an input): renumbers the rows that hold elements
 * 0, 1, 2, ... and keeps the map back to y in the sort permutation (slot 100); must be the first operator.
 * y keeps its length (as_matrix_y_rows); its entries for the removed rows are the zeros every SpMV clears y to. */
int as_matrix_remove_empty_rows(as_matrix *m);
int64_t as_matrix_y_rows(const as_matrix *m);
/* out = {rows, cols, nnz, origin_nnz, number of dense sub-blocks, is_sorted, is_compressed, wave} */
int as_matrix_info(const as_matrix *m, uint64_t out[8]);
/* key "val_copy_from_zero_quirk": 1 reproduces op_manager.cc:1081,1086 (sub-block values copied from offset 0) */
int as_matrix_set_option(as_matrix *m, const char *key, long value);
/* writes the current COO as .mtx.coo text (data_prepare.py output format) */
int as_matrix_write_coo_file(const as_matrix *m, const char *path);
/* writes the current COO as the binary cache that as_matrix_from_binary_file reads */
int as_matrix_write_binary_file(const as_matrix *m, const char *path);

/* ---- operator graph: exe_graph.cc:1443-2340 execute_exe_*_node, :2795
 * execute_exe_node_in_compressed_sub_matrix.  sub = -1 for dense-view nodes.
 *   COMPRESSED_ROW_PADDING          scalars = {multiply, padding_row_length}
 *   COMPRESSED_THREAD_LEVEL_NNZ_DIV scalars = {TLB_nnz_num}
 *   COMPRESSED_THREAD_LEVEL_COL_DIV list = TLB size of every WLB
 *   COMPRESSED_TBLOCK_LEVEL_ROW_DIV list = row count of every BLB
 *   COMPRESSED_TBLOCK_LEVEL_COL_DIV / WARP_LEVEL_ROW_DIV / WARP_LEVEL_COL_DIV
 *                                   counts[i] = number of entries of parent i, list = all entries, concatenated
 *   COMPRESSED_BLOCK_SORT           list = sort_block_index_arr: the BLBs whose rows are sorted by falling length
 *                                   (op_manager.cc:4104 compressed_block_sort; the reference has the operator and its
 *                                   templates read the permutation, but no node executor); right after the BLB
 *                                   level is made; an empty list = every BLB
 *   DENSE_ROW_COARSE_SORT           list = bin_row_nnz_low_bound
 *   DENSE_ROW_DIV                   list = row_div_position
 *   COMPRESS, COMPRESSED_THREAD_LEVEL_ROW_DIV   no parameters                                       */
int as_execute_node(as_matrix *m, int node_type, int64_t sub, const long *scalars, int n_scalars, const uint64_t *list,
                    uint64_t n_list, const uint64_t *counts, uint64_t n_counts);
/* parameter_set_strategy.cc:193-592 execute_*_param_strategy followed by the node itself.
 * p = the scalar knobs of the strategy in declaration order (parameter_set_strategy.hpp:24-110). */
int as_execute_strategy(as_matrix *m, int strategy, int64_t sub, const long p[4]);
/* default_auto_tuner.cc:384-447 execute_default_div_to_complete_each_level_blocking */
int as_complete_blocking(as_matrix *m, int64_t sub);

/* ---- introspection of the constructed format (what upstream dumps with
 * struct.cc:1657 print_arr_to_file_with_data_type).  Returns the array length
 * (copies min(len, cap) values into out when out != NULL), -1 if the array is
 * absent (NULL upstream), -2 on error. */
int64_t as_matrix_get_u64(const as_matrix *m, int64_t sub, int slot, int field, uint64_t *out, uint64_t cap, int *dtype);
int64_t as_matrix_get_f64(const as_matrix *m, int64_t sub, int which, double *out, uint64_t cap);


/* =====================================================================================
 * Kernel templates and the code builder (code_builder.hpp:60-189; every *_op.hpp).
 * One template per compressed sub-matrix: init_<T>_template re-lays the format out for its
 * kernel, try_all_compress replaces metadata arrays that follow a closed form
 * (arr_optimization.cc), code_of_template_kernal emits the HIP source of spmv_<sub>.
 * ===================================================================================== */

/* code_builder.cc:16 init_code_builder.  The matrix must stay alive while templates are set. */
as_builder *as_builder_create(const as_matrix *m);
void as_builder_free(as_builder *b);
/* is_supported_by_<T>(matrix, sub) of every *_op.hpp -> 1 / 0, <0 error */
int as_template_is_supported(const as_matrix *m, int64_t sub, int template_type);
/* init_<T>_template + add_template_to_builder (code_builder.hpp:160) */
int as_builder_set_template(as_builder *b, int64_t sub, int template_type);
/* compress_template_in_builder (code_builder.cc:2323) = try_all_compress of the template; 1 if anything compressed */
int as_builder_compress(as_builder *b, int64_t sub);
/* launch parameters of the template node (exe_graph.hpp:411-475); 0 leaves a value unchanged.
 * vec_width (1/2/4 TLBs or elements per lane and load) has no upstream counterpart. */
int as_builder_set_launch(as_builder *b, int64_t sub, long tblock_num, long thread_num_in_block,
                          long thread_num_of_row_reduce, long vec_width);
/* No counterpart in the reference.  Stores the columns of sub-matrix `sub` as 16-bit differences to the number of
 * the unit that reads them (2 bytes per element instead of 4), for banded matrices that are not sorted; only the
 * ELL template (AS_DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS).  1 = done (upload again), 0 = not applicable and
 * nothing changed (another template, or an element farther than 32767 columns from its unit), -1 error. */
int as_builder_set_relative_columns(as_builder *b, int64_t sub);
/* No counterpart in the reference.  One step further for stencils: when the elements of every unit lie on the same
 * few diagonals (as many as a unit has slots), every element is moved to the slot of its diagonal, the kernel
 * computes the column (unit number + the slot's offset) and reads no column array.  Same return values; the
 * offsets appear as scalars diagonal_offset_<k> in as_template_describe. */
int as_builder_set_diagonal_columns(as_builder *b, int64_t sub);
/* No counterpart in the reference.  Tile template (AS_SHARED_MEMORY_TILE_TEMPLATE) only: the template is built
 * again in its column-run form -- a lane of eight elements stores the first column of up to four runs of
 * consecutive columns and one byte of run starts, 9 bytes instead of 16 -- for matrices of dense blocks or dense
 * rows.  A lane that would need a fifth run is closed with zero-valued elements.  1 = done (upload again; the
 * launch setting is kept), 0 = nothing changed (another template, or the element stream would not get shorter
 * by 2 %), -1 error. */
int as_builder_set_column_runs(as_builder *b, int64_t sub);
/* No counterpart in the reference.  Tile template (AS_SHARED_MEMORY_TILE_TEMPLATE) only: the template is built
 * again under row ownership -- the elements are taken row group by row group (inside a group window by window of
 * x, from the group's own first column), every row group belongs to one workgroup, which keeps the group's row
 * sums in LDS across its windows and stores the rows to y at the end: no atomics, no table of places, no clear of y.  For matrices of many row groups that meet few column slices
 * each (banded matrices).  1 = done (upload again; the launch setting and the column-run form are kept), 0 =
 * nothing changed (another template, the form is in place, a column band of the matrix, slice copies that would
 * move more than a quarter of the element stream, or row groups too few or too uneven to fill the device),
 * -1 error. */
int as_builder_set_row_ownership(as_builder *b, int64_t sub);
/* No counterpart in the reference.  Tile template under row ownership only: where the rows of the sub-matrix come
 * in blocks of `rows_per_block` (2, 3 or 4) consecutive rows that hold the same columns (the dense blocks of a FEM
 * matrix), the template is built again with a block of rows as one piece of the stream: the columns, the lane
 * word and the reads of x are those of the block's first row, an element is one value per row.  The row group's
 * height must be a multiple of the block.  1 = done (upload again; launch setting, column-run form and row
 * ownership are kept), 0 = nothing changed (another template or form, rows that do not come in such blocks),
 * -1 error. */
int as_builder_set_row_blocks(as_builder *b, int64_t sub, int rows_per_block);
int as_builder_get_launch(as_builder *b, int64_t sub, long out[4]);
/* arrays of a template by upstream field name (what store_template_data writes to data_source/<id>/<name>).
 * "col_index_arr" and every metadata array here, "val_arr" through as_template_get_f64.
 * compress_type receives the arr_compress_type ordinal (arr_optimization.hpp:10-18). */
int64_t as_template_get_u64(as_builder *b, int64_t sub, const char *name, uint64_t *out, uint64_t cap, int *dtype,
                            int *compress_type);
int64_t as_template_get_f64(as_builder *b, int64_t sub, double *out, uint64_t cap);
/* "key=value" lines: template type, scalars (effective_TLB_num, is_atom_add, ...), "array:<name>=<dtype>,<len>,<compress>" */
const char *as_template_describe(as_builder *b, int64_t sub);
/* code_builder.cc:1322 code_of_template_kernal for every sub-matrix + shared preamble: the HIP module source */
const char *as_builder_kernel_source(as_builder *b);
/* executor.cc:61 compile_spmv_code: hipRTC for gfx950 (needs no GPU) */
int as_builder_compile(as_builder *b);
/* code_builder.cc:1248 code_of_write_template_data_to_gpu: module load + arrays into HBM */
int as_builder_upload(as_builder *b, int device);
/* y = A x, host vectors in the matrix value type.  y is cleared first by a fill kernel where the graph needs it
 * (as_builder_clears_y): a kernel adds into y with atomics, or some row of y is stored by no kernel.  Graphs whose
 * kernels store every row exactly once (ELL / SELL strips, the two-kernel LDS templates) launch no clear; whatever
 * y held before the call is overwritten either way.  The reference's generated program clears y with
 * cudaMemset before its timing loop only (code_builder.cc:1524-1557). */
int as_builder_spmv(as_builder *b, const void *x_host, void *y_host);
/* same on device pointers the caller owns */
int as_builder_spmv_device(as_builder *b, const void *x_dev, void *y_dev);
/* 1 when an SpMV of the builder's current templates starts with a clear of y, 0 when it does not; <0 error */
int as_builder_clears_y(as_builder *b);
/* Enqueue only: the launches of as_builder_spmv_device on a stream of the caller (a hipStream_t passed as a plain
 * pointer; NULL = HIP's default stream), no wait for the GPU -- the loop of the reference's generated program,
 * which launches spmv_<id><<<..., stream>>> repetition after repetition and synchronises once
 * (code_builder.cc:1517-1557).  With concurrent strip kernels (serial launch off) the strips' own streams fork from
 * and join the caller's stream by events.  The call may compile and load the module when the builder changed since
 * its upload (then it is no call for a capturing stream); as_builder_spmv_device is this call on the builder's own
 * stream (as_builder_stream) followed by a wait for that stream. */
int as_builder_spmv_device_async(as_builder *b, const void *x_dev, void *y_dev, void *stream);
/* the builder's own stream (a hipStream_t), on which the blocking calls and the timing calls launch */
void *as_builder_stream(as_builder *b);
/* No counterpart in the reference.  as_builder_spmv_device for callers that cannot allocate device memory (tight
 * serving loops, harnesses that forbid hipMalloc; code under HIP graph capture uses the _async twin below, since
 * this one waits for the GPU): the call compiles, loads and allocates nothing.  The builder must have been uploaded and not changed since (else an error), and the scratch
 * arrays of its kernels (row sums of a sorted tile strip, the products of the product-bin template) are 256-byte
 * aligned pieces of one static device array of AS_STATIC_SCRATCH_BYTES that the library holds on every GPU it has
 * uploaded to, until the process ends.  A graph whose kernels need more scratch than that
 * (as_builder_static_scratch_need) is rejected with an error: use as_builder_spmv_device for it.  All calls on
 * one GPU share the array, which keeps what the last call left (the pieces that must start at zero are cleared
 * by a fill kernel at the start of the call): calls that overlap on one GPU race. */
#define AS_STATIC_SCRATCH_BYTES (64u << 20)
int as_builder_spmv_device_no_alloc(as_builder *b, const void *x_dev, void *y_dev);
/* the same, enqueued on a stream of the caller without waiting for the GPU: nothing is compiled, loaded or
 * allocated and y and the scratch pieces are cleared by fill kernels (no memset node), so the call can be recorded
 * by a stream capture and replayed as a HIP graph (x_dev, y_dev and the builder's arrays must then stay where they
 * are).  Same limits and the same shared static array as above. */
int as_builder_spmv_device_no_alloc_async(as_builder *b, const void *x_dev, void *y_dev, void *stream);
/* bytes of the static scratch array the kernels of the builder's current templates would use (0: none) */
int64_t as_builder_static_scratch_need(as_builder *b);
/* 0 (default): the kernels of the sub-matrices run concurrently, one stream each (code_builder.cc:1517-1518);
 * 1: one after the other on the caller's stream.  No counterpart in the reference. */
int as_builder_set_serial_launch(as_builder *b, int serial);
/* With serial launch: the finish kernel of a tile-template strip (the move of its row sums from the scratch vector
 * to their places in y) is not launched where the strip after it has the product-bin template; the first
 * workgroups of that template's first kernel, which does not touch y, do the move instead.  1 (default): on;
 * 0: every template launches its own kernels.  Measurements of one sub-matrix alone always use its own kernels.
 * as_builder_finish_carrier: the sub-matrix whose first kernel carries the finish of `sub` under the builder's
 * current templates and settings, or -1.  No counterpart in the reference. */
int as_builder_set_finish_carry(as_builder *b, int on);
int as_builder_finish_carrier(as_builder *b, uint64_t sub, int64_t *carrier);
/* With a carried finish and the same workgroup size in both strips (default on): the first kernels of the two
 * strips are ONE launch -- every workgroup runs a trip of the tile strip and then trips of the product-bin strip, so
 * the end of the one and the start of the other overlap CU by CU instead of meeting at a kernel boundary -- and the
 * tile strip's rows are moved to y by the first workgroups of the product-bin strip's second kernel.  An SpMV of
 * such a graph is two launches.  0: every strip launches its first kernel itself.  No counterpart in the
 * reference, whose generated program launches one kernel per sub-matrix (code_builder.cc:1517-1549). */
int as_builder_set_fuse_launches(as_builder *b, int on);
/* 1 when the first kernel of `sub` is run by the first kernel of the strip behind it (so `sub` launches nothing of
 * its own in a whole SpMV), 0 when not, <0 on error */
int as_builder_launch_is_fused(as_builder *b, uint64_t sub);
/* `reps` back-to-back launches of the kernels of one sub-matrix only, timed with events on the launch stream;
 * also returns what that kernel's roofline figure is computed from: the bytes of its format arrays (padded
 * col + val + passed metadata), the rows of its strip and whether it accumulates y atomically.  No
 * counterpart in the reference (it times whole programs, code_builder.cc:1524-1557). */
int as_builder_time_sub_matrix(as_builder *b, int64_t sub, uint64_t reps, float *time_ms, uint64_t *format_bytes,
                               uint64_t *rows, int *atom);
/* the same for one of the two kernels of a sub-matrix whose template has two (pass 1 = spmv_<sub>, 2 =
 * spmv_<sub>_finish), launched alone `reps` times: a timing aid, y is not meaningful afterwards.  Fails when
 * the template has a single kernel.  No counterpart in the reference. */
int as_builder_time_sub_matrix_pass(as_builder *b, int64_t sub, int pass, uint64_t reps, float *time_ms);
/* The library keeps the code objects it compiled in this process, by module source (no counterpart in the
 * reference, which compiles every candidate with nvcc from a file: code_builder.cc:1463-1500): entries held and compilations answered from them. */
int as_kernel_cache_stats(uint64_t *entries, uint64_t *hits);
/* What the format builders and the search assume about the GPU: compute units, LDS a workgroup may take (both
 * read from the GPU at the first upload or search, which refuse a GPU that is not a gfx950; MI355X values until
 * then), XCDs and L2 bytes per XCD (fixed for gfx950).  The reference keeps the like in global_config.json
 * (e.g. its thread and shared-memory limits read by default_auto_tuner.cc).  from_device: 1 once read or set. */
int as_device_facts(uint64_t *cu_num, uint64_t *lds_bytes, uint64_t *xcd_num, uint64_t *l2_bytes_per_xcd, int *from_device);
/* read them from GPU `device` now (done implicitly by upload and search) */
int as_device_facts_read(int device);
/* formats for a GPU that cannot be asked (another partition mode; tests): 0 keeps a value */
int as_device_facts_set(uint64_t cu_num, uint64_t lds_bytes);
/* back to the MI355X values; the next upload or search asks its GPU again */
int as_device_facts_reset(void);
/* fill the builder's own x (used by the timing calls) */
int as_builder_set_x(as_builder *b, const void *x_host);
/* `reps` launches timed with events; gflops = 2 * origin_nnz * reps / time (code_builder.cc:1557).
 * sync_each_launch = 1 reproduces the upstream loop "kernel; cudaDeviceSynchronize" (code_builder.cc:1524-1557). */
int as_builder_time(as_builder *b, uint64_t reps, int sync_each_launch, float *time_ms, float *gflops);
/* bytes one SpMV moves with the chosen format: padded col+val, passed metadata, the kernels' scratch arrays written
 * and read back (2 x as_builder_scratch_bytes), x once, y once (twice where y is cleared first) */
int64_t as_builder_algorithmic_bytes(as_builder *b);
/* bytes of the scratch arrays of the kernels of sub-matrix `sub` (-1: of all): intermediate results the kernels write
 * and read back (products, row sums), which the format's own bytes count twice and a count of the format arrays,
 * x and y alone leaves out.  No counterpart in the reference. */
int64_t as_builder_scratch_bytes(as_builder *b, int64_t sub);
/* executor.hpp:12 part_execute_code_builder: run only the listed sub-matrices (n_ids = 0: all), `repeat` launches,
 * synchronising after each; repeat = 0 takes the reference's own count, 185.2e9 / (padded elements of the listed
 * sub-matrices), at least 2 (executor.cc:247-255).  Returns 0 and (time_ms for all launches, gflops), <0 on
 * failure (upstream: bool false) */
int as_part_execute_code_builder(as_builder *b, const int64_t *sub_matrix_ids, uint64_t n_ids, uint64_t repeat,
                                 float *time_ms, float *gflops);
/* executor.hpp:19 execute_code_builder: final run sized to about `seconds` (executor.cc:191-208) */
int as_execute_code_builder(as_builder *b, double seconds, uint64_t *repeat_out, float *time_ms, float *gflops);

/* arr_optimization.cc:6-420: try one compressor on an array (type = arr_compress_type ordinal;
 * param = cycle for CYCLE_LINEAR, max branches for BRANCH).  1 = pattern found,
 * out = {coefficient, intercept, constant, cycle, branches}. */
int as_compress_array(const uint64_t *values, uint64_t n, int type, uint64_t param, uint64_t out[5], uint64_t *eval,
                      char *code, uint64_t code_cap);
/* wave-level reduction helpers of the generated kernels, run on one wavefront (test hook) */
int as_selftest_group_sum(int device, int lanes, int is_double, const double *in, double *dpp_out, double *shfl_out);
/* segmented sum along the lanes of one wavefront (sorted keys), as the tile kernel uses it (test hook) */
int as_selftest_segmented_sum(int device, int is_double, const unsigned *key, const double *in, double *sum_out,
                              double *tail_out);
/* plain copy kernel `as_copy_words` of a known size (bytes read + bytes written per launch): calibrates the
 * FETCH_SIZE / WRITE_SIZE counters that the profiles of the SpMV kernels are scaled by */
int as_selftest_copy(int device, uint64_t bytes, int reps, float *ms_per_launch);

/* =====================================================================================
 * Search (whilte_list_path_impl.cc:5041 find_best_graph_of_white_list_strategy, default_auto_tuner.cc,
 * search_strategy.cc, param_enumerater.cc) and the best-graph report (whilte_list_path_impl.cc:4150,
 * parameter_set_strategy.cc:1119-1345, exe_graph.cc:3317, main.cc:646-663).
 * ===================================================================================== */
typedef struct as_search_result as_search_result;
typedef struct as_search_options {
  double total_time_s;           /* main.cc:634 init_search_strategy(10, 32400); 0 -> 120 */
  uint64_t struggle_step_num;    /* 0 -> 10 */
  double padding_rate_up_bound;  /* global_config.json PADDING_RATE_UP_BOUND; 0 -> 4 */
  int device;
  double timed_region_ms;        /* per candidate after warm-up; 0 -> 20 */
  const char *checkpoint_dir;    /* best_result_of_strategy{1,2,3} (whilte_list_path_impl.cc:5395-5412); NULL -> none */
  int verbose;                   /* candidate log also to stderr */
  int only_dense_strategy;       /* 0 all, 1/2/3 one dense-view strategy */
  int remove_empty_rows;         /* 0: an input with rows that hold no element is an error, as in the reference
                                  * (main.cc:604-621); 1: such rows are removed before the first operator */
  int general_templates;         /* 1: the two general templates DIRECT_ATOM / SHARED_MEMORY (direct_atom_op.cc,
                                  * shared_memory_op.cc), which the reference keeps out of its white list, are
                                  * searched as well (skeletons G1, G2) */
  int skip_verification;         /* no counterpart in the reference, which times candidates without looking at
                                  * their result.  0: every candidate runs once on x[j] = 1 + j % 7 and its y is compared
                                  * with a host CSR product for that x before it is timed; one that differs is logged,
                                  * counted as failed and cannot win.  1: candidates are only timed */
} as_search_options;
/* `input` = the matrix as read (no operator applied); its wave is the wave of every candidate */
as_search_result *as_find_best_graph(const as_matrix *input, const as_search_options *opt);
void as_search_free(as_search_result *r);
/* the best graph in test.log form: strategy nodes, "sub_matrix_id:i", kernel nodes */
const char *as_search_report(const as_search_result *r);
/* everything upstream prints while searching + "gflops:/time:" + report + "finish search" */
const char *as_search_log(const as_search_result *r);
/* The best graph as numbers, in the layout as_graph_report takes (dense nodes, then per sub-matrix its nodes and
 * its kernel node); returns how many numbers there are.  What main.cc:644 keeps as
 * dense_view_matrix_and_compressed_sub_block_exe_graph_and_template_t best_graph. */
int64_t as_search_best_graph(const as_search_result *r, long *desc, uint64_t cap);
/* out = {gflops, time_ms, candidates, failed candidates, seconds, seconds to best, sub-matrices, dense strategy} */
int as_search_stats(const as_search_result *r, double out[8]);
/* whilte_list_path_impl.cc:5318 execute_dense_view_matrix_and_compressed_sub_block_exe_graph_and_template:
 * rebuild the best format from `input`; the returned builder owns its matrix and is ready for as_builder_upload */
as_builder *as_search_build_best(const as_search_result *r, const as_matrix *input);

/* pieces of the search and of the report, one at a time (test hooks):
 * param_enumerater.cc:199 set_param_combination_to_next over n integer knobs (knob 0 fastest): every combination,
 * row-major in out; returns their number */
int64_t as_selftest_param_enumerator(int n, const long *low, const long *up, const long *step, long *out, uint64_t cap);
/* search_strategy.cc:24 continue_search(strategy, gflops) fed a series of candidate results without a time limit;
 * go[i] = 1 while the search would go on after candidate i */
int as_selftest_search_strategy(uint64_t struggle_step_num, const float *gflops, int n, int *go);
/* parameter_set_strategy.cc:1309 convert_stategy_node_to_string of one strategy node with knobs p; returns the text length */
int64_t as_strategy_report(int strategy, const long p[4], char *out, uint64_t cap);
/* exe_graph.cc:3317 convert_template_node_to_string of one kernel node */
int64_t as_template_node_report(int template_type, long tblock_num, long thread_num_in_block, long thread_num_of_row_reduce,
                                char *out, uint64_t cap);
/* whilte_list_path_impl.cc:4150-4228 convert_dense_view_matrix_and_compressed_sub_block_exe_graph_and_template_to_string_safety
 * of a whole operator graph: the text as_search_report returns for a search's best graph, here for a graph given
 * as numbers.  desc = n_dense, n_dense x (strategy, p0..p3), n_sub, then per sub-matrix: n_nodes, n_nodes x
 * (strategy, p0..p3), template type, tblock_num, thread_num_in_block, thread_num_of_row_reduce; the knobs of the
 * input node (DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT) are element count, value type, largest column index,
 * largest row index.  with_frame != 0: with the lines main.cc:646-657 prints around it ("gflops:", "time:", the
 * graph and an empty line or "error", "finish search"), which is the tail of as_search_log.  Returns the text length. */
int64_t as_graph_report(const long *desc, int64_t n_desc, int with_frame, float gflops, float time_ms, char *out,
                        uint64_t cap);

/* =====================================================================================
 * Thin HIP layer: what upstream reaches through system("./make_template.sh") (nvcc) and
 * system("./a.out") (executor.cc:6-104) and through the cudaMalloc / cudaMemcpy / kernel-launch /
 * gettimeofday text it generates (code_builder.cc:1471-1575).  Plain C types, status int,
 * caller-owned buffers.
 * ===================================================================================== */
const char *as_hip_last_error(void);
int as_hip_device_count(void);
int as_hip_init(int device);                                   /* cudaSetDevice(DEFAULT_DEVICE_ID), code_builder.cc:1489 */
/* no counterpart in the reference: address (on `device`) and size of the library's static scratch array, see
 * as_builder_spmv_device_no_alloc; looked up once per device, later calls return the kept pointer */
int as_hip_static_scratch(int device, void **ptr, uint64_t *bytes);
int as_hip_device_info(int device, char *name, int name_cap, int *cu_count, int *wave_size, uint64_t *lds_per_block,
                       uint64_t *global_mem);
/* hipRTC: HIP source -> gfx950 code object (malloc'ed, release with as_hip_free_host); needs no GPU */
int as_hip_compile(const char *src, const char *arch, const char *const *opts, int n_opts, void **code,
                   uint64_t *code_size, char **log);
void as_hip_free_host(void *p);
int as_hip_module_load(const void *code, void **module);
int as_hip_module_unload(void *module);
int as_hip_get_kernel(void *module, const char *name, void **fn);   /* "spmv_<sub_matrix_id>" */
int as_hip_alloc(void **p, uint64_t bytes);
int as_hip_free(void *p);
int as_hip_h2d(void *dst, const void *src, uint64_t bytes);
int as_hip_d2h(void *dst, const void *src, uint64_t bytes);
int as_hip_memset_async(void *dst, int value, uint64_t bytes, void *stream);
int as_hip_stream_create(void **stream);                       /* one stream per sub-matrix, code_builder.cc:1517 */
int as_hip_stream_destroy(void *stream);
int as_hip_stream_sync(void *stream);
int as_hip_device_sync(void);
int as_hip_event_create(void **ev);
int as_hip_event_destroy(void *ev);
int as_hip_event_record(void *ev, void *stream);
int as_hip_event_sync(void *ev);
int as_hip_event_elapsed_ms(void *start, void *stop, float *ms);
int as_hip_stream_wait_event(void *stream, void *ev);
/* stream capture into an executable graph and its replay (hipStreamBeginCapture / EndCapture / hipGraphInstantiate /
 * hipGraphLaunch): for callers that replay a fixed launch sequence; no counterpart in the reference */
int as_hip_graph_capture_begin(void *stream);
int as_hip_graph_capture_end(void *stream, void **graph_exec);
int as_hip_graph_launch(void *graph_exec, void *stream);
int as_hip_graph_destroy(void *graph_exec);
/* free and total device memory of the current GPU (hipMemGetInfo) */
int as_hip_mem_info(uint64_t *free_bytes, uint64_t *total_bytes);
int as_hip_launch(void *fn, unsigned grid, unsigned block, unsigned lds_bytes, void *stream, void **args);

#ifdef __cplusplus
}
#endif
#endif /* ALPHASPARSE_AMD_H */
