// SHARED_MEMORY_TEMPLATE_WARP_COMPRESS: SELL-like storage (one TLB size per
// BLB, column-major inside the BLB) with rows cut into several TLBs.  A
// workgroup owns a BLB: lanes compute TLB partials into LDS, then groups of R
// lanes (R = thread_num_of_row_reduce) add the partials of one row, driven by
// the CSR array row_offset_in_thread_tmp_result.  Format arrays follow upstream
// init_shared_memory_template_warp_compress (shared_memory_op_warp_compress.cc:198-533);
// unlike upstream (loop bound block_num - 1, :472) the last BLB is re-laid-out too.
#include "templates.hpp"

namespace asx {
namespace tpl_shared_memory_warp_compress {

static uint64_t lds_capacity(DType val_dtype) { return 65536 / (uint64_t)dtype_size(val_dtype) - 64; }

// is_supported_by_shared_memory_template_warp_compress (:535-718); the LDS
// bound is the 64 KB a gfx950 workgroup can allocate (upstream: 48000 - 50 entries)
bool is_supported(const Matrix &m, uint64_t sub) {
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &bl = *cb.read_index[2], &wl = *cb.read_index[3], &tl = *cb.read_index[4];
  if (tl.row_number.present) return false;
  bool many = false, first = true;
  uint64_t last_row = 0, max_tlb = 0;
  for (uint64_t b = 0; b < bl.block_num; b++) {
    if (b > 0 && bl.first_row[b] == bl.first_row[b - 1]) return false;
    uint64_t w0 = bl.index_arr[b], w1 = bl.index_arr[b + 1];
    max_tlb = std::max(max_tlb, wl.index_arr[w1] - wl.index_arr[w0]);
    for (uint64_t w = w0; w < w1; w++) {
      if (tl.coo_block_size[w] != tl.coo_block_size[w0]) return false;
      for (uint64_t t = wl.index_arr[w]; t < wl.index_arr[w + 1]; t++) {
        uint64_t r = bl.first_row[b] + wl.first_row[w] + tl.first_row[t];
        if (!first && r == last_row) many = true;
        first = false;
        last_row = r;
      }
    }
  }
  uint64_t max_row = bl.first_row[0] + bl.row_number[0] - 1;
  for (uint64_t b = 1; b < bl.block_num; b++) {
    if (bl.first_row[b] <= max_row) return false;
    max_row = std::max(max_row, bl.first_row[b] + bl.row_number[b] - 1);
  }
  return many && max_tlb <= lds_capacity(m.val_dtype);
}

std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  AS_CHECK(is_supported(m, sub), "format is not supported by SHARED_MEMORY_TEMPLATE_WARP_COMPRESS");
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &bl = *cb.read_index[2], &wl = *cb.read_index[3], &tl = *cb.read_index[4];
  auto t = std::make_unique<Template>();
  init_template_common(*t, SHARED_MEMORY_TEMPLATE_WARP_COMPRESS, m, sub);
  t->is_atom_add = sub_block_is_col_restricted(m, sub);
  t->scalar["effective_row_num"] = m.items[sub].max_row - m.items[sub].min_row + 1;
  uint64_t total_rows = bl.max_row - bl.min_row + 1;
  std::vector<uint64_t> row = global_row_of_each_TLB(cb);
  std::vector<uint64_t> offs(total_rows + 1, 0);
  for (uint64_t r : row) {
    AS_CHECK(r < total_rows, "TLB row outside the sub-matrix");
    offs[r + 1]++;
  }
  for (uint64_t r = 0; r < total_rows; r++) offs[r + 1] += offs[r];
  std::vector<uint64_t> tlb_size, tlb_begin;
  uint64_t max_tlb = 0;
  for (uint64_t b = 0; b < bl.block_num; b++) {
    tlb_size.push_back(tl.coo_block_size[bl.index_arr[b]]);
    tlb_begin.push_back(wl.index_arr[bl.index_arr[b]]);
  }
  tlb_begin.push_back(wl.index_arr[wl.block_num]);
  for (uint64_t b = 0; b < bl.block_num; b++) max_tlb = std::max(max_tlb, tlb_begin[b + 1] - tlb_begin[b]);
  t->scalar["max_TLB_num_in_block"] = max_tlb;

  const std::vector<uint64_t> &pcol = cb.read_index[5]->index_arr.v;
  const ValVec &pval = *cb.padding_val;
  t->col_index_arr.assign(std::vector<uint64_t>(pcol.size()), cb.read_index[5]->index_arr.dt);
  t->val_arr.resize(pval.size());
  for (uint64_t b = 0; b < bl.block_num; b++) {
    uint64_t nz0 = bl.coo_begin[b], n = tlb_begin[b + 1] - tlb_begin[b], s = tlb_size[b];
    AS_CHECK(n > 0 && nz0 + n * s <= pval.size(), "BLB offsets do not match the padded arrays");
    for (uint64_t i = 0; i < n; i++)
      for (uint64_t k = 0; k < s; k++) {
        t->col_index_arr.v[nz0 + i + k * n] = pcol[nz0 + i * s + k];
        t->val_arr[nz0 + i + k * n] = pval[nz0 + i * s + k];
      }
  }
  auto add = [&](const char *name, std::vector<uint64_t> v, DType dt) {
    TArr a;
    a.name = name;
    a.a.assign(std::move(v), dt);
    t->arrays.push_back(std::move(a));
  };
  uint64_t last = offs.back();
  add("row_offset_in_thread_tmp_result", std::move(offs), suitable_dtype(last));
  std::vector<uint64_t> bfr(bl.first_row.v.begin(), bl.first_row.v.begin() + bl.block_num);
  bfr.push_back(total_rows);
  add("block_first_row_index", std::move(bfr), suitable_dtype(total_rows));
  uint64_t last_tlb = tlb_begin.back();
  add("block_begin_thread_index_offset", std::move(tlb_begin), suitable_dtype(last_tlb));
  add("thread_block_size_in_block", std::move(tlb_size), tl.coo_block_size.dt);
  add("block_nz_begin_offset", std::vector<uint64_t>(bl.coo_begin.v.begin(), bl.coo_begin.v.begin() + bl.block_num),
      bl.coo_begin.dt);
  if (m.sorted_row_index.present) {
    t->global_sort_index = true;
    add("row_index_before_sort", m.sorted_row_index.v, m.sorted_row_index.dt);
  } else if (cb.y_write_index.present) {  // rows sorted inside BLBs: the permutation is relative to the sub-matrix
    add("row_index_before_sort", cb.y_write_index.v, cb.y_write_index.dt);
  }
  tpl_shared_memory_warp_compress::set_default_launch(*t);
  return t;
}

// try_all_compress (:2334-2354)
void try_all_compress(Template &t) {
  TArr &o = *t.find("block_begin_thread_index_offset");
  if (!o.c.active()) init_linear_compressor(o.a, o.c, true);
  TArr &s = *t.find("thread_block_size_in_block");
  if (!s.c.active() && !init_constant_compressor(s.a, s.c, true) && s.a.size() > 2) init_branch_compressor(s.a, s.c, 5);
  for (const char *n : {"block_nz_begin_offset", "block_first_row_index", "row_offset_in_thread_tmp_result"}) {
    TArr &a = *t.find(n);
    if (!a.c.active()) init_linear_compressor(a.a, a.c, true);
  }
}

void set_default_launch(Template &t) {
  uint64_t lanes = t.sc("max_TLB_num_in_block");
  if (t.thread_num_in_block == 0) t.thread_num_in_block = std::min<uint64_t>(1024, std::max<uint64_t>(64, (lanes + 63) / 64 * 64));
  t.tblock_num = std::min<uint64_t>(t.arr("thread_block_size_in_block").a.size(), (1ull << 31) - 1);
  if (t.thread_num_of_row_reduce == 0) t.thread_num_of_row_reduce = 1;
}

std::string kernel_source(const Template &t) {
  AS_CHECK(t.val_arr.size() < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
  const uint64_t R = t.thread_num_of_row_reduce;
  AS_CHECK(R >= 1 && R <= 64 && (R & (R - 1)) == 0, "thread_num_of_row_reduce must be a power of two <= 64");
  const std::string vt = value_type_name(t);
  const std::string id = std::to_string(t.sub), B = std::to_string(t.thread_num_in_block), Rs = std::to_string(R);
  const std::string fc = std::to_string(t.kernal_first_col_index) + "u";
  const uint64_t nblb = t.arr("thread_block_size_in_block").a.size();
  std::string s;
  s += "extern \"C\" __global__ void __launch_bounds__(" + B + ") spmv_" + id + "(" + kernel_signature(t) + ")\n{\n";
  s += "  __shared__ " + vt + " thread_tmp_result[" + std::to_string(t.sc("max_TLB_num_in_block")) + "];\n";
  s += "  for (unsigned int blb = as_xcd_block_index(); blb < " + std::to_string(nblb) + "u; blb += gridDim.x)\n  {\n";
  s += "    unsigned int next_blb = blb + 1u, block_first_nz, first_tlb, next_first_tlb, tlb_size, first_row, next_first_row;\n";
  s += "    " + code_of_meta_read(t, "block_nz_begin_offset", "block_first_nz", "blb");
  s += "    " + code_of_meta_read(t, "block_begin_thread_index_offset", "first_tlb", "blb");
  s += "    " + code_of_meta_read(t, "block_begin_thread_index_offset", "next_first_tlb", "next_blb");
  s += "    " + code_of_meta_read(t, "thread_block_size_in_block", "tlb_size", "blb");
  s += "    " + code_of_meta_read(t, "block_first_row_index", "first_row", "blb");
  s += "    " + code_of_meta_read(t, "block_first_row_index", "next_first_row", "next_blb");
  s += "    const unsigned int tlb_num = next_first_tlb - first_tlb;\n";
  s += "    for (unsigned int t = threadIdx.x; t < tlb_num; t += " + B + "u)\n    {\n";
  s += "      " + vt + " acc = 0;\n      unsigned int nz = block_first_nz + t;\n";
  s += "      #pragma unroll 4\n      for (unsigned int k = 0; k < tlb_size; k++, nz += tlb_num)\n";
  s += "        acc += as_ldnt(val_arr + nz) * device_x_arr[" + fc + " + (unsigned int)as_ldnt(col_index_arr + nz)];\n";
  s += "      thread_tmp_result[t] = acc;\n    }\n";
  s += "    as_barrier();\n";
  s += "    for (unsigned int row = first_row + threadIdx.x / " + Rs + "u; row < next_first_row; row += " + B + "u / " + Rs + "u)\n    {\n";
  s += "      unsigned int next_row = row + 1u, res_begin, res_end;\n";
  s += "      " + code_of_meta_read(t, "row_offset_in_thread_tmp_result", "res_begin", "row");
  s += "      " + code_of_meta_read(t, "row_offset_in_thread_tmp_result", "res_end", "next_row");
  s += "      " + vt + " sum = 0;\n";
  s += "      for (unsigned int i = res_begin + (threadIdx.x % " + Rs + "u); i < res_end; i += " + Rs + "u) sum += thread_tmp_result[i - first_tlb];\n";
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

}  // namespace tpl_shared_memory_warp_compress
}  // namespace asx
