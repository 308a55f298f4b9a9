// SHARED_MEMORY_LONG_ROW_TEMPLATE: one BLB = one piece of one (long) row.  A
// workgroup streams its piece with 128-bit loads (4 consecutive elements per
// lane), reduces inside each wavefront with DPP, combines the wavefront sums
// through LDS and writes (or, when pieces share a row, atomically adds) one
// value.  Format arrays follow upstream init_shared_memory_long_row_template
// (shared_memory_long_row_op.cc:3-210).
#include "templates.hpp"

namespace asx {
namespace tpl_shared_memory_long_row {

// is_supported_by_shared_memory_long_row_template (:212-248)
bool is_supported(const Matrix &m, uint64_t sub) {
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &bl = *cb.read_index[2], &tl = *cb.read_index[4];
  if (tl.row_number.present) return false;
  for (uint64_t b = 0; b < bl.block_num; b++)
    if (bl.row_number[b] != 1) return false;
  return true;
}

std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  AS_CHECK(is_supported(m, sub), "every BLB must hold exactly one row");
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &bl = *cb.read_index[2], &wl = *cb.read_index[3], &tl = *cb.read_index[4];
  auto t = std::make_unique<Template>();
  init_template_common(*t, SHARED_MEMORY_LONG_ROW_TEMPLATE, m, sub);
  bool atom = sub_block_is_col_restricted(m, sub);
  for (uint64_t b = 0; b < bl.block_num; b++) {
    if (b + 1 < bl.block_num && bl.first_row[b] == bl.first_row[b + 1]) atom = true;
    AS_CHECK((bl.coo_begin[b + 1] - bl.coo_begin[b]) % m.wave == 0, "BLB nnz must be a multiple of the wave size");
  }
  AS_CHECK(bl.coo_begin[bl.block_num] == cb.padding_val->size(), "BLB offsets do not cover the padded arrays");
  for (uint64_t w = 0; w < wl.block_num; w++) AS_CHECK(tl.coo_block_size[w] == 1, "TLB size must be 1");
  t->is_atom_add = atom;

  std::vector<uint64_t> row(bl.first_row.v.begin(), bl.first_row.v.begin() + bl.block_num);
  // rows appended by COMPRESSED_ROW_PADDING never reach this template upstream
  // (the template is only searched on unpadded graphs); they are masked here anyway
  uint64_t effective = effective_unit_num(m, sub, row);
  t->global_sort_index = apply_global_sort(m, sub, row, effective);
  t->scalar["effective_BLB_num"] = effective;
  uint64_t max_nnz = 0;
  for (uint64_t b = 0; b < bl.block_num; b++) max_nnz = std::max(max_nnz, bl.coo_begin[b + 1] - bl.coo_begin[b]);
  t->scalar["max_BLB_nnz"] = max_nnz;

  TArr r, o;
  r.name = "row_index_of_block_level_block";
  uint64_t mx = *std::max_element(row.begin(), row.end());
  r.a.assign(std::move(row), suitable_dtype(mx));
  o.name = "block_nz_begin_offset";
  o.a = bl.coo_begin;
  t->arrays.push_back(std::move(r));
  t->arrays.push_back(std::move(o));
  t->val_arr = *cb.staggered_val;
  t->col_index_arr = cb.read_index[6]->index_arr;
  tpl_shared_memory_long_row::set_default_launch(*t);
  return t;
}

// try_all_compress (:971-985)
void try_all_compress(Template &t) {
  TArr &r = *t.find("row_index_of_block_level_block");
  if (!r.c.active() && !init_linear_compressor(r.a, r.c, true)) init_cycle_increase_compressor(r.a, r.c, true);
  TArr &o = *t.find("block_nz_begin_offset");
  if (!o.c.active()) init_linear_compressor(o.a, o.c, true);
}

void set_default_launch(Template &t) {
  // a lane covers 4 elements per trip; aim at ~4 trips for the longest piece
  uint64_t lanes = (t.sc("max_BLB_nnz") + 15) / 16;
  if (t.thread_num_in_block == 0) t.thread_num_in_block = std::min<uint64_t>(1024, std::max<uint64_t>(64, (lanes + 63) / 64 * 64));
  t.tblock_num = std::min<uint64_t>(t.sc("effective_BLB_num"), (1ull << 31) - 1);
  if (t.tblock_num == 0) t.tblock_num = 1;
}

std::string kernel_source(const Template &t) {
  const std::string vt = value_type_name(t), ct = dtype_c_name(t.col_index_arr.dt);
  const uint64_t eff = t.sc("effective_BLB_num");
  AS_CHECK(t.val_arr.size() < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
  AS_CHECK(t.wave == 64, "kernel is written for 64-lane wavefronts; build the format with wave = 64");
  const std::string id = std::to_string(t.sub), B = std::to_string(t.thread_num_in_block);
  const std::string fc = std::to_string(t.kernal_first_col_index) + "u";
  const uint64_t waves = t.thread_num_in_block / 64;
  std::string s;
  s += "extern \"C\" __global__ void __launch_bounds__(" + B + ") spmv_" + id + "(" + kernel_signature(t) + ")\n{\n";
  // 16 bytes of values per lane and load (four floats or two doubles): the 64 lanes of a load read one contiguous KB
  const std::string V = std::to_string(16 / dtype_size(t.val_dtype));
  s += "  typedef " + vt + " valv_t __attribute__((ext_vector_type(" + V + ")));\n";
  s += "  typedef " + ct + " colv_t __attribute__((ext_vector_type(" + V + ")));\n";
  if (waves > 1) s += "  __shared__ " + vt + " wave_sum[" + std::to_string(waves) + "];\n";
  s += "  for (unsigned int blb = as_xcd_block_index(); blb < " + std::to_string(eff) + "u; blb += gridDim.x)\n  {\n";
  s += "    unsigned int next_blb = blb + 1u, nz_begin, nz_end;\n";
  s += "    " + code_of_meta_read(t, "block_nz_begin_offset", "nz_begin", "blb");
  s += "    " + code_of_meta_read(t, "block_nz_begin_offset", "nz_end", "next_blb");
  s += "    " + vt + " acc = 0;\n";
  // piece lengths are multiples of 64, so a lane's group of elements never straddles the end
  s += "    for (unsigned int nz = nz_begin + threadIdx.x * " + V + "u; nz < nz_end; nz += " + B + "u * " + V + "u)\n    {\n";
  s += "      valv_t a = as_ldnt((const valv_t *)(val_arr + nz));\n";
  s += "      colv_t c = as_ldnt((const colv_t *)(col_index_arr + nz));\n";
  s += "      #pragma unroll\n      for (int j = 0; j < " + V + "; j++) acc += a[j] * device_x_arr[" + fc + " + (unsigned int)c[j]];\n";
  s += "    }\n";
  s += "    acc = as_wave_sum(acc);\n";
  if (waves > 1) {
    s += "    if ((threadIdx.x & 63u) == 63u) wave_sum[threadIdx.x >> 6] = acc;\n";
    s += "    as_barrier();\n";
    s += "    if (threadIdx.x == 0)\n    {\n      acc = 0;\n";
    s += "      #pragma unroll\n      for (int w = 0; w < " + std::to_string(waves) + "; w++) acc += wave_sum[w];\n";
  } else {
    s += "    if (threadIdx.x == 63u)\n    {\n";
  }
  s += "      unsigned int global_row_index;\n      " +
       code_of_meta_read(t, "row_index_of_block_level_block", "global_row_index", "blb");
  if (!t.global_sort_index && t.kernal_first_row_index != 0)
    s += "      global_row_index += " + std::to_string(t.kernal_first_row_index) + "u;\n";
  s += t.is_atom_add ? "      as_atomic_add(device_y_arr + global_row_index, acc);\n"
                     : "      as_stnt(device_y_arr + global_row_index, acc);\n";
  s += "    }\n";
  if (waves > 1) s += "    as_barrier();\n";
  s += "  }\n}\n";
  return s;
}

}  // namespace tpl_shared_memory_long_row
}  // namespace asx
