// Code builder + executor: one kernel template per compressed sub-matrix, the
// HIP module generated from them, device residency of the arrays, launches and
// timing.  Host-side counterpart of upstream code_builder.hpp:60-189 and
// executor.hpp:12-24, with the text-file / nvcc / a.out hand-off replaced by
// in-memory arrays, hipRTC and in-process launches.
#pragma once
#include "templates.hpp"

namespace asx {

struct DeviceBuf {
  void *ptr = nullptr;
  size_t bytes = 0;
};

struct SubKernel {
  std::unique_ptr<Template> tpl;
  std::vector<DeviceBuf> meta;  // one per passed metadata array, kernel-argument order
  DeviceBuf val, col, scratch;
  void *fn = nullptr;
  void *finish_fn = nullptr;  // spmv_<sub>_finish when the template has one
  void *stream = nullptr;
  void *done = nullptr;  // event
  bool uploaded = false;
};

struct Builder {
  const Matrix *matrix = nullptr;  // not owned; must outlive template initialisation
  uint64_t rows = 0, cols = 0, origin_nnz = 0;
  bool rows_compacted = false;     // remove_empty_rows ran: y has rows that no kernel stores
  DType val_dtype = FLOAT;
  std::vector<SubKernel> subs;     // index = sub-matrix id; tpl == nullptr until set
  std::string source;
  std::vector<char> code;
  void *module = nullptr;
  void *zero_fn = nullptr;
  void *main_stream = nullptr, *start_ev = nullptr, *t0 = nullptr, *t1 = nullptr;
  DeviceBuf x, y;
  void *static_scratch = nullptr;  // the library's static scratch array on this GPU (launch_spmv_no_alloc)
  uint64_t static_scratch_bytes = 0;
  bool device_ready = false;
  bool module_stale = true;  // source changed since the module was loaded
  // false: every sub-matrix kernel runs on its own stream, all at once; true: one after the other on
  // the caller's stream (kernels that each fill the machine only get in each other's way)
  bool serial_launch = false;
  // With serial_launch: the finish kernel of a tile-template strip is not launched where the strip after it has a
  // product-bin template; the first workgroups of that template's first kernel do its work instead (see
  // assign_finish_carriers).  false: every template launches its own kernels.
  bool carry_finish = true;
  // With a carried finish and workgroups of the same size in both strips: the first kernels of the two strips are
  // one launch (Template::fused_trips).  false: two launches.
  bool fuse_launches = true;
  // >= 0: launches and timing cover the kernels of this sub-matrix only (per-kernel measurement)
  int64_t only_sub = -1;
  int only_pass = 0;  // with only_sub: 1 = the first kernel alone, 2 = the finish kernel alone, 0 = both
  std::string compile_log;
  ~Builder();
};

std::unique_ptr<Builder> init_code_builder(const Matrix &m);                       // code_builder.cc:16
void add_template_to_builder(Builder &b, uint64_t sub, TemplateType type);          // init_<T>_template + add
bool compress_template_in_builder(Builder &b, uint64_t sub);                         // code_builder.cc:2323
// make_columns_relative on the template of one sub-matrix; its arrays are uploaded again at the next upload
bool set_relative_columns(Builder &b, uint64_t sub);
// make_columns_diagonal on the template of one sub-matrix; same rules
bool set_diagonal_columns(Builder &b, uint64_t sub);
// The tile template of a sub-matrix built at once in a combination of its forms (row ownership, blocks of rows as
// pieces, column runs where they make the element stream at least 2 % shorter): what the search measures first on a
// banded matrix whose rows come in blocks, instead of walking there one form at a time.  false (builder unchanged)
// where the combination does not apply.
bool add_tile_template_variant_to_builder(Builder &b, uint64_t sub, bool column_runs_if_shorter, bool own_rows, uint64_t row_block);
// Rebuilds the tile template of a sub-matrix in its column-run form (init_tile_template_with_column_runs) and
// keeps it when the element stream gets shorter by at least 2 %; false (template unchanged) otherwise, or when
// the sub-matrix has another template.  The launch setting is kept.
bool set_column_runs(Builder &b, uint64_t sub);
// Rebuilds the tile template of a sub-matrix under row ownership (init_tile_template_variant; the column-run form
// is kept when it is in place); false (template unchanged) when the sub-matrix has another template, the form
// is in place already or it does not fit the sub-matrix.  The launch setting is kept.
bool set_row_ownership(Builder &b, uint64_t sub);
// Tile template under row ownership: blocks of `rows_per_block` (2-4) consecutive rows that hold the same columns
// stored as one piece (one set of columns and lane words for the block).  false where the rows do not come in
// such blocks, the row group's height is not a multiple of the block, or the form is in place.
bool set_row_blocks(Builder &b, uint64_t sub, uint64_t rows_per_block);
// Whole module: preamble + every spmv_<sub> (code_of_kernal_define, build_main_file's kernel part)
std::string build_module_source(const Builder &b);
void compile_builder(Builder &b);                 // hipRTC, no GPU needed (compile_spmv_code, executor.cc:61)
// code objects kept by module source, and how often a compilation was answered from them
void code_cache_stats(uint64_t &entries, uint64_t &hits);
void load_and_upload(Builder &b, int device);     // module load + arrays to HBM (code_of_write_template_data_to_gpu)
// True when y has to be cleared before the kernels run: a kernel adds into y (atomics), a row of y belongs to
// no kernel (rows removed by remove_empty_rows, a sub-matrix without template) or holds no element.  Graphs whose
// kernels store every row exactly once (ELL / SELL strips, the two-kernel LDS templates) skip the clear.
bool y_needs_clear(const Builder &b);
// Zeroes the scratch array of one sub-matrix's kernels (after its first kernel ran without its finish kernel).
void clear_scratch(Builder &b, uint64_t sub);
// Decides which finish kernels are carried by the strip launched next (Template::carried of the carrying
// template), from the templates, serial_launch and carry_finish; build_module_source calls it.  Returns the
// sub-matrix whose first kernel carries the finish of `sub`, or -1.
int64_t assign_finish_carriers(const Builder &b, uint64_t sub = ~0ull);
// y = A x on device buffers already holding x; y is cleared first where y_needs_clear says so.
void launch_spmv(Builder &b, const void *x_dev, void *y_dev);
// the same on a stream of the caller (a hipStream_t; nullptr = the default stream): enqueues and returns
void launch_spmv(Builder &b, const void *x_dev, void *y_dev, void *stream);
// The same SpMV for callers that must not allocate device memory: nothing is compiled, loaded or allocated
// (the builder must be uploaded), and the kernels' scratch arrays are pieces of the library's static scratch
// array on this GPU instead of the builder's own.  Fails when the graph needs more scratch than the array holds.
// Calls that overlap on one GPU share the array and race.
void launch_spmv_no_alloc(Builder &b, const void *x_dev, void *y_dev);
void launch_spmv_no_alloc(Builder &b, const void *x_dev, void *y_dev, void *stream);
uint64_t static_scratch_need(const Builder &b);  // bytes of the static array the graph's kernels would use
void spmv_host(Builder &b, const void *x_host, void *y_host);
// Timing: `reps` launches of all kernels.  sync_each_launch reproduces the
// upstream loop (kernel; cudaDeviceSynchronize, code_builder.cc:1524-1557).
// Every repetition is what launch_spmv issues (the clear of y included where needed).
// Returns ms for all reps; gflops = 2 * origin_nnz * reps / time.
void time_spmv(Builder &b, uint64_t reps, bool sync_each_launch, float &time_ms, float &gflops);
// Bytes one SpMV moves with the chosen format (padded col/val + passed
// metadata + x once + y once, y twice when a kernel accumulates atomically).
uint64_t builder_algorithmic_bytes(const Builder &b);
void release_device(Builder &b);
void invalidate_module(Builder &b);  // after a launch-parameter change
// Drop the template of one sub-matrix (and its device arrays).
void remove_template_from_builder(Builder &b, uint64_t sub);

std::vector<uint8_t> narrow_bytes(const IArr &a);
std::vector<uint8_t> narrow_values(const ValVec &v, DType dt);

}  // namespace asx
