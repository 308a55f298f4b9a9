// The two WARP_TOTAL_RED templates: every WLB is (a piece of) one row and is
// reduced by one 64-lane wavefront with DPP.
//
//  DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE  the wavefront's last lane writes or
//      atomically adds the sum to y (upstream direct_atom_total_warp_reduce_op.cc:3-247)
//  SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE  WLB sums of a BLB are staged in LDS
//      and added per row by groups of R lanes, R = thread_num_of_row_reduce
//      (upstream shared_memory_total_warp_reduce_op.cc:3-258)
//
// Elements of a WLB may be read in any order (it is a single row), so both
// kernels stream the interleaved arrays with 1/2/4-element loads per lane.
#include "templates.hpp"

namespace asx {
namespace {

// WLB -> (row relative to the sub-matrix, absolute first element); checks one row per WLB
void walk_wlbs(const CompressedBlock &cb, unsigned wave, std::vector<uint64_t> &row, std::vector<uint64_t> &first_nz) {
  const Index &bl = *cb.read_index[2], &wl = *cb.read_index[3];
  row.assign(wl.block_num, 0);
  first_nz.assign(wl.block_num + 1, 0);
  for (uint64_t b = 0; b < bl.block_num; b++)
    for (uint64_t w = bl.index_arr[b]; w < bl.index_arr[b + 1]; w++) {
      AS_CHECK(wl.row_number[w] == 1, "every WLB must hold exactly one row");
      row[w] = bl.first_row[b] + wl.first_row[w];
      first_nz[w] = bl.coo_begin[b] + wl.coo_begin[w];
      if (w > 0) AS_CHECK((first_nz[w] - first_nz[w - 1]) % wave == 0, "WLB nnz must be a multiple of the wave size");
    }
  first_nz[wl.block_num] = cb.padding_val->size();
  AS_CHECK((first_nz[wl.block_num] - first_nz[wl.block_num - 1]) % wave == 0, "WLB nnz must be a multiple of the wave size");
}

bool one_row_wlbs(const CompressedBlock &cb) {
  const Index &wl = *cb.read_index[3], &tl = *cb.read_index[4];
  if (tl.row_number.present) return false;
  for (uint64_t w = 0; w < wl.block_num; w++)
    if (wl.row_number[w] != 1) return false;
  return true;
}

// lane-strided dot product of one WLB [nz_begin, nz_end) followed by the wave sum
std::string code_of_wlb_dot(const Template &t, const std::string &ind) {
  const std::string vt = value_type_name(t), V = std::to_string(t.vec_width);
  const std::string fc = std::to_string(t.kernal_first_col_index) + "u";
  std::string s;
  s += ind + vt + " acc = 0;\n";
  s += ind + "for (unsigned int nz = nz_begin + lane * " + V + "u; nz < nz_end; nz += 64u * " + V + "u)\n" + ind + "{\n";
  if (t.vec_width == 1) {
    s += ind + "  " + vt + " a = as_ldnt(val_arr + nz);\n" + ind + "  unsigned int c = as_ldnt(col_index_arr + nz);\n";
    s += ind + "  acc += a * device_x_arr[" + fc + " + c];\n";
  } else {
    s += ind + "  valv_t a = as_ldnt((const valv_t *)(val_arr + nz));\n";
    s += ind + "  colv_t c = as_ldnt((const colv_t *)(col_index_arr + nz));\n";
    s += ind + "  #pragma unroll\n" + ind + "  for (int j = 0; j < " + V + "; j++) acc += a[j] * device_x_arr[" + fc +
         " + (unsigned int)c[j]];\n";
  }
  s += ind + "}\n" + ind + "acc = as_wave_sum(acc);\n";
  return s;
}

std::string vec_typedefs(const Template &t) {
  const std::string V = std::to_string(t.vec_width);
  return "  typedef " + value_type_name(t) + " valv_t __attribute__((ext_vector_type(" + V + ")));\n  typedef " +
         dtype_c_name(t.col_index_arr.dt) + " colv_t __attribute__((ext_vector_type(" + V + ")));\n";
}

}  // namespace

// ===========================================================================
namespace tpl_direct_atom_total_warp_reduce {

bool is_supported(const Matrix &m, uint64_t sub) { return one_row_wlbs(*m.items[sub].cb); }

std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  const CompressedBlock &cb = *m.items[sub].cb;
  AS_CHECK(is_supported(m, sub), "every WLB must hold exactly one row");
  auto t = std::make_unique<Template>();
  init_template_common(*t, DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE, m, sub);
  std::vector<uint64_t> row, first_nz;
  walk_wlbs(cb, m.wave, row, first_nz);
  bool atom = sub_block_is_col_restricted(m, sub);
  for (size_t w = 1; w < row.size() && !atom; w++) atom = row[w] == row[w - 1];
  t->is_atom_add = atom;
  uint64_t effective = effective_unit_num(m, sub, row);
  t->global_sort_index = apply_global_sort(m, sub, row, effective);
  t->scalar["effective_WLB_num"] = effective;
  TArr r, o;
  r.name = "global_row_index_of_warp_level_block";
  uint64_t mx = *std::max_element(row.begin(), row.end());
  r.a.assign(std::move(row), suitable_dtype(mx));
  o.name = "global_warp_nz_begin_offset";
  o.a.assign(std::move(first_nz), suitable_dtype(cb.padding_val->size() + 1));
  t->arrays.push_back(std::move(r));
  t->arrays.push_back(std::move(o));
  t->val_arr = *cb.staggered_val;
  t->col_index_arr = cb.read_index[6]->index_arr;
  tpl_direct_atom_total_warp_reduce::set_default_launch(*t);
  return t;
}

// try_all_compress (:1063-1077)
void try_all_compress(Template &t) {
  TArr &r = *t.find("global_row_index_of_warp_level_block");
  if (!r.c.active() && !init_linear_compressor(r.a, r.c, true)) init_cycle_increase_compressor(r.a, r.c, true);
  TArr &o = *t.find("global_warp_nz_begin_offset");
  if (!o.c.active()) init_linear_compressor(o.a, o.c, true);
}

void set_default_launch(Template &t) {
  if (t.thread_num_in_block == 0) t.thread_num_in_block = 256;
  uint64_t waves = t.thread_num_in_block / 64;
  t.tblock_num = std::max<uint64_t>(1, std::min<uint64_t>((t.sc("effective_WLB_num") + waves - 1) / waves, (1ull << 31) - 1));
}

std::string kernel_source(const Template &t) {
  AS_CHECK(t.wave == 64, "kernel is written for 64-lane wavefronts; build the format with wave = 64");
  AS_CHECK(t.val_arr.size() < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
  const std::string id = std::to_string(t.sub), B = std::to_string(t.thread_num_in_block);
  const std::string waves = std::to_string(t.thread_num_in_block / 64);
  std::string s;
  s += "extern \"C\" __global__ void __launch_bounds__(" + B + ") spmv_" + id + "(" + kernel_signature(t) + ")\n{\n";
  s += vec_typedefs(t);
  s += "  const unsigned int lane = threadIdx.x & 63u;\n";
  s += "  for (unsigned int wlb = as_xcd_block_index() * " + waves + "u + (threadIdx.x >> 6); wlb < " +
       std::to_string(t.sc("effective_WLB_num")) + "u; wlb += gridDim.x * " + waves + "u)\n  {\n";
  s += "    unsigned int next_wlb = wlb + 1u, nz_begin, nz_end;\n";
  s += "    " + code_of_meta_read(t, "global_warp_nz_begin_offset", "nz_begin", "wlb");
  s += "    " + code_of_meta_read(t, "global_warp_nz_begin_offset", "nz_end", "next_wlb");
  s += code_of_wlb_dot(t, "    ");
  s += "    if (lane == 63u)\n    {\n      unsigned int global_row_index;\n      " +
       code_of_meta_read(t, "global_row_index_of_warp_level_block", "global_row_index", "wlb");
  if (!t.global_sort_index && t.kernal_first_row_index != 0)
    s += "      global_row_index += " + std::to_string(t.kernal_first_row_index) + "u;\n";
  s += t.is_atom_add ? "      as_atomic_add(device_y_arr + global_row_index, acc);\n"
                     : "      as_stnt(device_y_arr + global_row_index, acc);\n";
  s += "    }\n  }\n}\n";
  return s;
}

}  // namespace tpl_direct_atom_total_warp_reduce

// ===========================================================================
namespace tpl_shared_memory_total_warp_reduce {

static uint64_t lds_capacity(DType val_dtype) { return 65536 / (uint64_t)dtype_size(val_dtype) - 8; }

// is_supported_by_shared_memory_total_warp_reduce_template (:260-394): BLB row
// ranges strictly increasing, one row per WLB, at least one row cut into
// several WLBs, and the WLB sums of a BLB fit the LDS of a workgroup (64 KB on
// gfx950; upstream bound: SHARED_MEM_TOTAL_SIZE - 5 entries).
bool is_supported(const Matrix &m, uint64_t sub) {
  const CompressedBlock &cb = *m.items[sub].cb;
  if (!one_row_wlbs(cb)) return false;
  const Index &bl = *cb.read_index[2], &wl = *cb.read_index[3];
  uint64_t max_row = bl.first_row[0] + bl.row_number[0] - 1;
  for (uint64_t b = 1; b < bl.block_num; b++) {
    if (bl.first_row[b] <= max_row) return false;
    max_row = std::max(max_row, bl.first_row[b] + bl.row_number[b] - 1);
  }
  bool many = false;
  for (uint64_t b = 0; b < bl.block_num; b++) {
    if (bl.index_arr[b + 1] - bl.index_arr[b] > lds_capacity(m.val_dtype)) return false;
    for (uint64_t w = bl.index_arr[b] + 1; w < bl.index_arr[b + 1]; w++)
      if (wl.first_row[w] == wl.first_row[w - 1]) many = true;
  }
  return many;
}

std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  AS_CHECK(is_supported(m, sub), "format is not supported by SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE");
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &bl = *cb.read_index[2];
  auto t = std::make_unique<Template>();
  init_template_common(*t, SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE, m, sub);
  t->is_atom_add = sub_block_is_col_restricted(m, sub);
  std::vector<uint64_t> row, first_nz;
  walk_wlbs(cb, m.wave, row, first_nz);
  uint64_t total_rows = cb.read_index[0]->max_row - cb.read_index[0]->min_row + 1;
  std::vector<uint64_t> offs(total_rows + 1, 0);
  for (uint64_t r : row) offs[r + 1]++;
  for (uint64_t r = 0; r < total_rows; r++) offs[r + 1] += offs[r];
  t->scalar["effective_row_num"] = m.items[sub].max_row - m.items[sub].min_row + 1;
  uint64_t max_wlb = 0;
  for (uint64_t b = 0; b < bl.block_num; b++) max_wlb = std::max(max_wlb, bl.index_arr[b + 1] - bl.index_arr[b]);
  t->scalar["max_WLB_num_in_block"] = max_wlb;

  auto add = [&](const char *name, std::vector<uint64_t> v, DType dt) {
    TArr a;
    a.name = name;
    a.a.assign(std::move(v), dt);
    t->arrays.push_back(std::move(a));
  };
  uint64_t last = offs.back();
  add("row_offset_in_warp_tmp_result", std::move(offs), suitable_dtype(last));
  std::vector<uint64_t> bfr(bl.first_row.v.begin(), bl.first_row.v.begin() + bl.block_num);
  bfr.push_back(total_rows);
  add("block_first_row_index", std::move(bfr), suitable_dtype(total_rows));
  add("block_begin_warp_index_offset", bl.index_arr.v, bl.index_arr.dt);
  uint64_t last_nz = first_nz.back();
  add("global_warp_block_first_nz", std::move(first_nz), suitable_dtype(last_nz));
  if (m.sorted_row_index.present) {
    t->global_sort_index = true;
    add("row_index_before_sort", m.sorted_row_index.v, m.sorted_row_index.dt);
  } else if (cb.y_write_index.present) {  // rows sorted inside BLBs: the permutation is relative to the sub-matrix
    add("row_index_before_sort", cb.y_write_index.v, cb.y_write_index.dt);
  }
  t->val_arr = *cb.staggered_val;
  t->col_index_arr = cb.read_index[6]->index_arr;
  tpl_shared_memory_total_warp_reduce::set_default_launch(*t);
  return t;
}

// try_all_compress (:1803-1820)
void try_all_compress(Template &t) {
  for (const char *n : {"block_begin_warp_index_offset", "row_offset_in_warp_tmp_result", "block_first_row_index",
                        "global_warp_block_first_nz"}) {
    TArr &a = *t.find(n);
    if (!a.c.active()) init_linear_compressor(a.a, a.c, true);
  }
}

void set_default_launch(Template &t) {
  uint64_t lanes = t.sc("max_WLB_num_in_block") * 64;
  if (t.thread_num_in_block == 0) t.thread_num_in_block = std::min<uint64_t>(1024, std::max<uint64_t>(64, lanes));
  t.tblock_num = std::min<uint64_t>(t.arr("block_first_row_index").a.size() - 1, (1ull << 31) - 1);
  if (t.thread_num_of_row_reduce == 0) t.thread_num_of_row_reduce = 1;
}

std::string kernel_source(const Template &t) {
  AS_CHECK(t.wave == 64, "kernel is written for 64-lane wavefronts; build the format with wave = 64");
  AS_CHECK(t.val_arr.size() < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
  const uint64_t R = t.thread_num_of_row_reduce;
  AS_CHECK(R >= 1 && R <= 64 && (R & (R - 1)) == 0, "thread_num_of_row_reduce must be a power of two <= 64");
  const std::string vt = value_type_name(t);
  const std::string id = std::to_string(t.sub), B = std::to_string(t.thread_num_in_block), Rs = std::to_string(R);
  const std::string waves = std::to_string(t.thread_num_in_block / 64);
  const uint64_t nblb = t.arr("block_first_row_index").a.size() - 1;
  std::string s;
  s += "extern \"C\" __global__ void __launch_bounds__(" + B + ") spmv_" + id + "(" + kernel_signature(t) + ")\n{\n";
  s += vec_typedefs(t);
  s += "  __shared__ " + vt + " warp_tmp_result[" + std::to_string(t.sc("max_WLB_num_in_block")) + "];\n";
  s += "  const unsigned int lane = threadIdx.x & 63u;\n";
  s += "  for (unsigned int blb = as_xcd_block_index(); blb < " + std::to_string(nblb) + "u; blb += gridDim.x)\n  {\n";
  s += "    unsigned int next_blb = blb + 1u, first_wlb, next_first_wlb, first_row, next_first_row;\n";
  s += "    " + code_of_meta_read(t, "block_begin_warp_index_offset", "first_wlb", "blb");
  s += "    " + code_of_meta_read(t, "block_begin_warp_index_offset", "next_first_wlb", "next_blb");
  s += "    " + code_of_meta_read(t, "block_first_row_index", "first_row", "blb");
  s += "    " + code_of_meta_read(t, "block_first_row_index", "next_first_row", "next_blb");
  s += "    for (unsigned int wlb = first_wlb + (threadIdx.x >> 6); wlb < next_first_wlb; wlb += " + waves + "u)\n    {\n";
  s += "      unsigned int next_wlb = wlb + 1u, nz_begin, nz_end;\n";
  s += "      " + code_of_meta_read(t, "global_warp_block_first_nz", "nz_begin", "wlb");
  s += "      " + code_of_meta_read(t, "global_warp_block_first_nz", "nz_end", "next_wlb");
  s += code_of_wlb_dot(t, "      ");
  s += "      if (lane == 63u) warp_tmp_result[wlb - first_wlb] = acc;\n    }\n";
  s += "    as_barrier();\n";
  // rows of the BLB: groups of R lanes add the WLB sums of one row
  s += "    for (unsigned int row = first_row + threadIdx.x / " + Rs + "u; row < next_first_row; row += " + B + "u / " + Rs + "u)\n    {\n";
  s += "      unsigned int next_row = row + 1u, res_begin, res_end;\n";
  s += "      " + code_of_meta_read(t, "row_offset_in_warp_tmp_result", "res_begin", "row");
  s += "      " + code_of_meta_read(t, "row_offset_in_warp_tmp_result", "res_end", "next_row");
  s += "      " + vt + " sum = 0;\n";
  s += "      for (unsigned int i = res_begin + (threadIdx.x % " + Rs + "u); i < res_end; i += " + Rs + "u) sum += warp_tmp_result[i - first_wlb];\n";
  s += "      sum = as_group_sum<" + Rs + ">(sum);\n";
  s += "      if ((threadIdx.x % " + Rs + "u) == " + Rs + "u - 1u && row < " + std::to_string(t.sc("effective_row_num")) +
       "u && res_end > res_begin)\n      {\n";
  if (t.local_sort_index && !t.global_sort_index)
    s += "        unsigned int global_row_index = row_index_before_sort[row] + " + std::to_string(t.kernal_first_row_index) + "u;\n";
  else
    s += "        unsigned int global_row_index = row + " + std::to_string(t.kernal_first_row_index) + "u;\n";
  if (t.global_sort_index) s += "        global_row_index = row_index_before_sort[global_row_index];\n";
  s += t.is_atom_add ? "        as_atomic_add(device_y_arr + global_row_index, sum);\n"
                     : "        as_stnt(device_y_arr + global_row_index, sum);\n";
  s += "      }\n    }\n";
  s += "    as_barrier();\n  }\n}\n";
  return s;
}

}  // namespace tpl_shared_memory_total_warp_reduce
}  // namespace asx
