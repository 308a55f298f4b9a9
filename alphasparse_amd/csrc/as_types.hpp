// Matrix data model of the SpMV format generator.
//
// Mirrors the upstream POD structs (struct.hpp:32-241: data_type,
// index_of_compress_block_t, compressed_block_t, dense_block_table_item_t,
// sparse_struct_t) with owned, typed C++17 containers instead of void*+tag
// arrays.  Every index array keeps its *logical* values as u64 together with
// the narrowed element type the upstream code would have chosen for it, so
// "bit-exact" means (values, dtype) equality; narrowing to bytes happens only
// at the export / device-upload boundary.
#pragma once
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace asx {

// Same ordinal values as upstream `enum data_type` (struct.hpp:32-47).
enum DType : int {
  CHAR, UNSIGNED_CHAR, SHORT, UNSIGNED_SHORT, INT, UNSIGNED_INT, LONG, UNSIGNED_LONG,
  LONG_LONG, UNSIGNED_LONG_LONG, FLOAT, DOUBLE, BOOL, NONE_DATA_TYPE
};

enum CompressedIndexType : int { COO, CSR, ELL, NO_INDEX };       // struct.hpp:14-20
enum IndexType : int { BLOCK_INDEX, ROW_INDEX, COL_INDEX };        // struct.hpp:23-28
enum IndexLevel : int { TBLOCK_LEVEL, WRAP_LEVEL, THREAD_LEVEL, OTHERS };  // struct.hpp:50-56

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};
#define AS_CHECK(cond, msg)                                                            \
  do {                                                                                 \
    if (!(cond)) throw ::asx::Error(std::string(__func__) + ": " + (msg));             \
  } while (0)

// find_most_suitable_data_type (op_manager.cc:1103-1134)
inline DType suitable_dtype(uint64_t max_value) {
  if (max_value <= 255ull) return UNSIGNED_CHAR;
  if (max_value <= 65535ull) return UNSIGNED_SHORT;
  if (max_value <= 4294967295ull) return UNSIGNED_INT;
  return UNSIGNED_LONG;
}
inline int dtype_size(DType t) {
  switch (t) {
    case CHAR: case UNSIGNED_CHAR: case BOOL: return 1;
    case SHORT: case UNSIGNED_SHORT: return 2;
    case INT: case UNSIGNED_INT: case FLOAT: return 4;
    case LONG: case UNSIGNED_LONG: case LONG_LONG: case UNSIGNED_LONG_LONG: case DOUBLE: return 8;
    default: return 0;
  }
}
const char *dtype_name(DType t);       // convert_data_type_to_string (struct.cc:740)
const char *dtype_c_name(DType t);     // element type spelled in generated kernel source

// An integer metadata / index array: logical values + upstream-chosen dtype.
struct IArr {
  DType dt = NONE_DATA_TYPE;
  std::vector<uint64_t> v;
  bool present = false;  // upstream pointer != NULL
  void assign(std::vector<uint64_t> vals, DType t) {
    v = std::move(vals);
    dt = t;
    present = true;
  }
  void clear() {
    v.clear();
    v.shrink_to_fit();
    dt = NONE_DATA_TYPE;
    present = false;
  }
  size_t size() const { return v.size(); }
  uint64_t operator[](size_t i) const { return v[i]; }
  uint64_t max_value() const {
    uint64_t m = 0;
    for (uint64_t x : v) m = x > m ? x : m;
    return m;
  }
  // Narrowest type that really holds the values, never narrower than `want`.
  // Used where an upstream max-tracking quirk would pick a type too small.
  static DType at_least(DType want, uint64_t real_max) {
    DType need = suitable_dtype(real_max);
    return dtype_size(need) > dtype_size(want) ? need : want;
  }
};

// One level of the compressed-view index hierarchy (index_of_compress_block_t).
struct Index {
  IndexLevel level = OTHERS;
  CompressedIndexType ctype = COO;
  IndexType itype = BLOCK_INDEX;
  uint64_t block_num = 0;
  uint64_t length = 0;
  IArr index_arr;              // COO payload, or CSR "first child" offsets
  IArr first_row;              // index_of_the_first_row_arr
  IArr row_number;             // row_number_of_block_arr
  IArr coo_begin;              // coo_begin_index_arr
  IArr coo_block_size;         // coo_block_size_arr
  uint64_t max_row = 0, min_row = 0, max_col = 0, min_col = 0;
};
using IndexPtr = std::shared_ptr<Index>;
using ValVec = std::vector<double>;  // fp32 values are held widened (exact)
using ValPtr = std::shared_ptr<ValVec>;

// compressed_block_t (struct.hpp:121-160)
struct CompressedBlock {
  std::vector<IndexPtr> read_index;
  bool share_row_with_other_block = false;
  bool share_row_with_other_warp = false;
  bool share_row_with_other_thread = false;
  DType val_dtype = FLOAT;
  ValPtr val;                // val_arr            (size == read_index[1]->length)
  ValPtr padding_val;        // padding_val_arr
  ValPtr staggered_val;      // staggered_padding_val_arr
  // compressed_block_sort (struct.hpp compressed_block_t::is_sorted, y_write_index[0]): the rows inside some BLBs
  // were re-ordered by length; y_write_index[row after the sort] = row before it, both relative to the sub-matrix
  bool is_sorted = false;
  IArr y_write_index;
  // Column slice width when the BLBs were cut at column slice boundaries
  // (COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE_PARAM_STRATEGY), else 0.
  uint64_t col_slice = 0;
  // Row group height when the BLBs are 2-D tiles (rows of one group x columns of one slice,
  // COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY), else 0.
  uint64_t row_group = 0;
  std::unique_ptr<CompressedBlock> clone() const;
};

// dense_block_table_item_t (struct.hpp:162-187)
struct DenseItem {
  uint64_t min_row = 0, max_row = 0, min_col = 0, max_col = 0;
  uint64_t begin_coo = 0, end_coo = 0;
  bool is_col_blocked = false;
  std::unique_ptr<CompressedBlock> cb;
};

// sparse_struct_t (struct.hpp:203-241) + the operator_manager binding.
struct Matrix {
  uint64_t rows = 0, cols = 0, nnz = 0, origin_nnz = 0;
  // Length of y.  Equal to `rows` unless remove_empty_rows renumbered the rows that hold elements
  // 0..rows-1; sorted_row_index then maps them back (and a later sort goes through that map).
  uint64_t y_rows = 0;
  bool rows_compacted = false;
  bool is_compressed = false, is_blocked = false, is_sorted = false;
  IArr sorted_row_index;                 // sorted_row_index[new] = old
  std::vector<DenseItem> items;          // block_coor_table.item_arr
  std::vector<uint64_t> coo_row, coo_col;
  ValVec coo_val;
  DType val_dtype = FLOAT;
  // Lane count the thread-level operators pad / interleave for.  32 reproduces
  // the upstream arrays bit for bit; 64 is the CDNA wavefront.
  unsigned wave = 64;
  // compress_dense_view upstream copies every sub-block's values from offset 0
  // of the global value array (op_manager.cc:1081,1086).  true = reproduce that
  // (only meaningful for all-equal values); false = copy from begin_coo.
  bool val_copy_from_zero_quirk = false;
  std::unique_ptr<Matrix> clone() const;  // val_copy_from_old_matrix_struct (struct.cc:392)
  // Trial isolation without copying the whole matrix: header fields, sort permutation and the
  // dense block table, but only the compressed view of `sub` (no global COO arrays).
  std::unique_ptr<Matrix> clone_for_sub(uint64_t sub) const;
  CompressedBlock &block(uint64_t sub) {
    AS_CHECK(sub < items.size() && items[sub].cb, "sub-matrix " + std::to_string(sub) + " is not compressed");
    return *items[sub].cb;
  }
};

}  // namespace asx
