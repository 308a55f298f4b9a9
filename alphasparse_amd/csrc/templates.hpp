// Kernel templates ("reduction operators"): for one compressed sub-matrix a
// template owns the device-side arrays (re-laid-out col/val + metadata), knows
// which metadata arrays follow a closed form, and emits the HIP source of its
// kernel `spmv_<sub>`.  One struct serves every template family; the family
// specific code lives in tpl_*.cc.
#pragma once
#include <algorithm>
#include <map>

#include "arr_optimization.hpp"
#include "as_types.hpp"

namespace asx {

// Same order as upstream `enum template_type` (code_builder.hpp:15-29).
enum TemplateType : int {
  DIRECT_ATOM_TEMPLATE, DIRECT_ATOM_TEMPLATE_WARP_COMPRESS, DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS,
  SHARED_MEMORY_TEMPLATE, SHARED_MEMORY_TEMPLATE_WARP_COMPRESS, SHARED_MEMORY_LONG_ROW_TEMPLATE,
  SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE, DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE,
  UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE, UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE,
  EMPTY_TEMPLATE, NONE_TEMPLATE,
  // no upstream counterpart (kept behind the upstream ordinals): one-row BLBs cut at column slice
  // boundaries, the slice of x staged in LDS
  SHARED_MEMORY_X_SLICE_TEMPLATE,
  // no upstream counterpart: 2-D tiles (row group x column slice), the slice of x and the row
  // group's sums staged in LDS
  SHARED_MEMORY_TILE_TEMPLATE,
  // no upstream counterpart: the same 2-D tiles in two passes -- products through an LDS-resident slice
  // of x streamed to scratch, then summed per row group in LDS (short rows, no gather from HBM)
  SHARED_MEMORY_PRODUCT_BIN_TEMPLATE,
  TEMPLATE_TYPE_COUNT
};
const char *convert_template_type_to_string(TemplateType t);  // code_builder.cc

// A metadata array of a template (+ its closed form once compressed away).
struct TArr {
  std::string name;
  IArr a;
  Compressor c;
  // false: host-side intermediate kept for inspection only (never uploaded,
  // not a kernel argument, not counted as traffic)
  bool on_device = true;
  bool passed() const { return on_device && !c.active(); }
};

struct Template {
  TemplateType type = NONE_TEMPLATE;
  uint64_t sub = 0;               // dense_block_index
  unsigned wave = 64;
  DType val_dtype = FLOAT;
  uint64_t matrix_rows = 0;       // dense_row_number of the whole matrix
  uint64_t matrix_cols = 0;       // dense_col_number of the whole matrix
  uint64_t kernal_first_row_index = 0, kernal_first_col_index = 0;
  bool is_atom_add = false;
  bool global_sort_index = false;
  // the rows inside BLBs were sorted (compressed_block_sort): row numbers go through y_write_index, which is
  // relative to the sub-matrix (upstream local_sort_index, e.g. direct_atom_op.cc:153-175)
  bool local_sort_index = false;
  // template specific scalars (effective_TLB_num, thread_block_size_in_block, ...)
  std::map<std::string, uint64_t> scalar;
  std::vector<TArr> arrays;       // metadata arrays, in kernel-argument order
  IArr col_index_arr;
  ValVec val_arr;
  uint64_t origin_nnz = 0;        // non-padding elements this kernel covers
  // elements of the compressed sub-matrix with the padding of its operators (compressed_block_t::padding_arr_size,
  // op_manager.cc:3789, 3933): what the executor sizes its default repeat count by (executor.cc:237)
  uint64_t padding_arr_size = 0;
  // launch parameters (template_node params, exe_graph.hpp:411-475)
  uint64_t tblock_num = 0, thread_num_in_block = 0, thread_num_of_row_reduce = 1;
  // Rows (or TLBs) handled per lane with one wide load; 1, 2 or 4.  An MI355X
  // tuning knob without upstream counterpart.
  unsigned vec_width = 1;
  // the columns are stored as 16-bit differences to the number of the unit (TLB) that reads them (no upstream
  // counterpart; banded matrices): see make_columns_relative
  bool col_relative = false;
  // not empty: element k of every unit lies at column (unit number + col_diagonal[k]) and no column array is
  // read at all (no upstream counterpart; stencils): see make_columns_diagonal
  std::vector<long> col_diagonal;
  // tile template: the columns of a lane's eight elements are stored as the first columns of up to four runs
  // of consecutive columns plus a byte of run starts (no upstream counterpart; dense blocks, dense rows): see
  // init_tile_template_with_column_runs
  bool col_runs = false;
  // tile template: every row group belongs to one workgroup, which keeps the group's row sums in LDS across the
  // slices and stores the rows to y at the end -- no atomics, no clear of y (no upstream counterpart; matrices of
  // many row groups that meet few slices each): see init_tile_template_variant
  bool own_rows = false;
  // tile template under row ownership: rows come in blocks of this many consecutive rows with the same columns and
  // are stored as such (1 = every row by itself): see init_tile_template_variant
  uint64_t row_block = 1;
  // Carried finish (set by the builder when it writes the module, see assign_finish_carriers): the first
  // `carried_blocks` workgroups of this template's first kernel do the work of the finish kernel of `carried`, the
  // template of the row strip launched before this one, and leave; the other workgroups number themselves from 0.
  // Not owned; nullptr = none.
  const Template *carried = nullptr;
  uint64_t carried_blocks = 0;
  // Fused launch (set by the builder together with `carried`, see assign_finish_carriers): this template's first
  // kernel runs the trips of the first kernel of `fused_trips` -- the template of the row strip in front of it, the
  // same as `carried` -- ahead of its own, workgroup by workgroup, so that strip launches nothing of its own; the
  // carried finish then moves to THIS template's finish kernel (everything of the strip in front must be done
  // before its row sums are read).  Not owned; nullptr = none.
  const Template *fused_trips = nullptr;
  // LDS the kernel asks for at launch (beyond its static __shared__ arrays)
  uint64_t dynamic_lds_bytes = 0;
  // Device scratch of the kernels (last argument `scratch_arr`): allocated and cleared once at upload; what
  // it holds between two SpMVs is the template's business (the tile template leaves it cleared).  0 = none.
  uint64_t scratch_bytes = 0;
  // true: the kernels rely on the scratch array holding zeros when an SpMV starts (the tile template adds row
  // sums into it and clears it again); false: every word that is read was written earlier in the same SpMV
  bool scratch_starts_zero = false;
  // > 0: a second kernel `spmv_<sub>_finish` with this many workgroups follows spmv_<sub> on the same
  // stream (same arguments)
  uint64_t finish_tblock_num = 0, finish_thread_num = 256, finish_lds_bytes = 0;
  // false: the kernels store every row of their strip of y exactly once and add to none, so y need not be
  // cleared for them (set by add_template_to_builder through template_needs_cleared_y)
  bool y_needs_clear = true;

  TArr *find(const std::string &n) {
    for (auto &t : arrays)
      if (t.name == n) return &t;
    return nullptr;
  }
  const TArr &arr(const std::string &n) const {
    for (auto &t : arrays)
      if (t.name == n) return t;
    throw Error("template has no array " + n);
  }
  uint64_t sc(const std::string &n) const {
    auto it = scalar.find(n);
    AS_CHECK(it != scalar.end(), "template has no scalar " + n);
    return it->second;
  }
};

// Bytes one SpMV with this template has to move: padded col + val, every
// metadata array still passed to the kernel, nothing for compressed ones.
uint64_t template_format_bytes(const Template &t);

// ---- shared helpers (tpl_common.cc) ---------------------------------------
// Row (relative to the sub-matrix) of every TLB: BLB first row + WLB first row
// + TLB first row, walking the three levels (e.g. direct_atom_op.cc:60-110).
std::vector<uint64_t> global_row_of_each_TLB(const CompressedBlock &cb);
// True if the dense block does not span all columns (partial sums need atomics).
bool sub_block_is_col_restricted(const Matrix &m, uint64_t sub);
// First TLB whose row lies in the rows appended by COMPRESSED_ROW_PADDING
// (upstream effective_TLB_num, e.g. direct_atom_op_warp_compress.cc:255-296).
uint64_t effective_unit_num(const Matrix &m, uint64_t sub, const std::vector<uint64_t> &unit_row);
// Map rows through the global sort permutation (sorted_row_index[new] = old)
// for the first `effective` units; returns whether a permutation was applied.
bool apply_global_sort(const Matrix &m, uint64_t sub, std::vector<uint64_t> &unit_row, uint64_t effective);
void init_template_common(Template &t, TemplateType type, const Matrix &m, uint64_t sub);
// True when the kernels of `t` add into y anywhere (atomics on shared rows, on rows that cross a tile) or when a
// row of the strip holds no element and is therefore stored by nobody: y must then be cleared before the launch.
bool template_needs_cleared_y(const Template &t, const Matrix &m, uint64_t sub);

// ---- per-family entry points ------------------------------------------------
// is_supported_by_<T>, init_<T>, try_all_compress, code_of_template_kernal,
// dispatched by type (upstream code_builder.cc:446-595, 1248-1469).
bool is_supported_by_template(TemplateType type, const Matrix &m, uint64_t sub);
std::unique_ptr<Template> init_template(TemplateType type, const Matrix &m, uint64_t sub);
void try_all_compress(Template &t);
// Default launch shape for a freshly initialised template.
void set_default_launch(Template &t);
// Re-encodes the column array as 16-bit differences to the reading unit's number where the template supports it
// and every difference fits; false (template unchanged) otherwise.  Only DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS.
bool make_columns_relative(Template &t);
// Goes one step further where every element of a unit lies on one of as many diagonals as the unit has slots
// (a stencil): the elements are put into the slot of their diagonal and the column array disappears.  false
// (template unchanged) otherwise.  Only DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS.
bool make_columns_diagonal(Template &t);
// SHARED_MEMORY_TILE_TEMPLATE built in its column-run form (Template::col_runs): same kernel family, 9 bytes of
// columns per lane of eight elements instead of 16 where consecutive elements lie in consecutive columns.  A
// lane that would hold more than four runs is closed with zero-valued elements, so the form exists for every
// matrix the template supports, and costs padding where columns are not consecutive: compare val_arr sizes.
std::unique_ptr<Template> init_tile_template_with_column_runs(const Matrix &m, uint64_t sub);
// SHARED_MEMORY_TILE_TEMPLATE in any combination of its two forms (column runs, row ownership); nullptr when row
// ownership is asked for and does not fit the sub-matrix: a column band of the matrix, slice copies that would
// move more than a quarter of the element stream's bytes, or trips (whole row groups) too uneven to fill the device.
// row_block = b > 1 (only under row ownership): b consecutive rows that hold the same columns share their columns,
// lane words and x reads; nullptr where some block of rows does not (or b does not divide the row group's height).
std::unique_ptr<Template> init_tile_template_variant(const Matrix &m, uint64_t sub, bool column_runs, bool own_rows,
                                                     uint64_t row_block = 1);
// Height (4, 3, 2, else 1) of the blocks of rows with equal columns that a tile-divided sub-matrix seems to be made
// of, judged from its first tile; what the search looks at before it tries init_tile_template_variant(.., row_block).
uint64_t tile_row_block_guess(const Matrix &m, uint64_t sub);
// Elements the tile template's stream would hold in the column-run form (lane-closing padding included), counted in
// one pass without building the template: what set_column_runs looks at before it builds anything.
uint64_t tile_column_run_stream_estimate(const Matrix &m, uint64_t sub);
// HIP source of `extern "C" __global__ void spmv_<sub>(...)`.
std::string code_of_template_kernal(const Template &t);
// Kernel arguments in order: names of the metadata arrays that are passed
// (not compressed away); val_arr, col_index_arr, device_x_arr, device_y_arr follow.
std::vector<std::string> kernel_array_args(const Template &t);

#define AS_DECLARE_TEMPLATE(ns)                                        \
  namespace ns {                                                       \
  bool is_supported(const Matrix &m, uint64_t sub);                    \
  std::unique_ptr<Template> init(const Matrix &m, uint64_t sub);       \
  void try_all_compress(Template &t);                                  \
  void set_default_launch(Template &t);                                \
  std::string kernel_source(const Template &t);                        \
  }
AS_DECLARE_TEMPLATE(tpl_direct_atom)
AS_DECLARE_TEMPLATE(tpl_direct_atom_warp_compress)
AS_DECLARE_TEMPLATE(tpl_direct_atom_warp_block_compress)
AS_DECLARE_TEMPLATE(tpl_shared_memory)
AS_DECLARE_TEMPLATE(tpl_shared_memory_warp_compress)
AS_DECLARE_TEMPLATE(tpl_shared_memory_long_row)
AS_DECLARE_TEMPLATE(tpl_shared_memory_total_warp_reduce)
AS_DECLARE_TEMPLATE(tpl_direct_atom_total_warp_reduce)
AS_DECLARE_TEMPLATE(tpl_unaligned_warp_reduce)
AS_DECLARE_TEMPLATE(tpl_unaligned_warp_reduce_with_warp_reduce)
AS_DECLARE_TEMPLATE(tpl_empty)
AS_DECLARE_TEMPLATE(tpl_shared_memory_x_slice)
AS_DECLARE_TEMPLATE(tpl_shared_memory_tile)
AS_DECLARE_TEMPLATE(tpl_shared_memory_product_bin)
#undef AS_DECLARE_TEMPLATE

// ---- source emission helpers (codegen.cc) ----------------------------------
// Preamble shared by every generated module: value/atomic helpers, wave64
// DPP reductions.
std::string kernel_module_preamble();
// "const <type>* __restrict__ <name>, " for every passed metadata array, then
// val/col/x/y.
std::string kernel_signature(const Template &t);
// the same with every parameter name behind `prefix` (a kernel that takes the arrays of two templates), and the
// matching argument list "prefix + name, ..." for a call
std::string kernel_signature(const Template &t, const std::string &prefix);
std::string kernel_arguments(const Template &t, const std::string &prefix);
// Name of the device function that holds the body of a template's first kernel, for templates whose trips another
// template's kernel can run (the tile template): (kernel_signature, unsigned as_block, unsigned as_grid).
std::string kernel_trips_function_name(const Template &t);
// A kernel that can carry another template's finish (Template::carried) appends carried_finish_signature to its
// parameters and opens its body with carried_finish_prologue: the code of the carrying workgroups, then the
// definitions of as_block / as_grid, the number of this workgroup among the kernel's own and how many those are.
// `threads` = the kernel's workgroup size.  Extra launch arguments in order: the carried template's scratch
// vector, its y_row_index array where that is passed, the number of its rows (0 = nothing to do this launch).
std::string carried_finish_signature(const Template &host);
std::string carried_finish_prologue(const Template &host, uint64_t threads);
bool carried_place_is_passed(const Template &guest);
// "<type> <var>;  <var> = name[idx] | closed form;" honouring compression.
std::string code_of_meta_read(const Template &t, const std::string &arr, const std::string &var,
                              const std::string &idx);
std::string value_type_name(const Template &t);
std::string y_row_type_name(const Template &t);

}  // namespace asx
