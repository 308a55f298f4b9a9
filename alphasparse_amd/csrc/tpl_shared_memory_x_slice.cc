// SHARED_MEMORY_X_SLICE_TEMPLATE (no upstream counterpart): long rows whose columns are spread
// over the whole vector.  Every BLB is a piece of one row that lies inside one column slice of
// `col_slice` columns (COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE_PARAM_STRATEGY); the BLBs are
// regrouped by slice, and a workgroup copies its slice of x into LDS once (128 KB of the 160 KB a
// CU has) and then serves every x read of its BLBs from there.  That replaces one L2 request per
// element -- what bounds gathers from a vector larger than L2 -- by coalesced streaming, and lets
// the column index shrink to 16 bits (an offset inside the slice).  BLB lengths are multiples of 64
// (the thread-level operator pads them), so the elements of a workgroup trip form a flat run of
// 64-element units, each inside one BLB: a wavefront streams four units per step (16 lanes x 4
// consecutive elements per unit, 128-bit value loads), sums each unit over its 16 lanes with DPP row
// operations and adds it to the unit's row with one atomic (rows are shared between slices and
// units, so y is always accumulated atomically).  No per-BLB control flow, no dependent loads.
#include "device_facts.hpp"
#include "templates.hpp"

namespace asx {
namespace tpl_shared_memory_x_slice {

// largest slice whose values fit the LDS budget of one workgroup (128 KB; 32 KB stay free)
static const unsigned kBatch = 4;  // steps of 4 units whose loads a wavefront keeps in flight together
static uint64_t max_slice(DType val_dtype) { return x_slice_bytes() / (uint64_t)dtype_size(val_dtype); }

bool is_supported(const Matrix &m, uint64_t sub) {
  const DenseItem &it = m.items[sub];
  const CompressedBlock &cb = *it.cb;
  const Index &bl = *cb.read_index[2], &wl = *cb.read_index[3], &tl = *cb.read_index[4];
  if (tl.row_number.present || cb.col_slice == 0 || cb.col_slice > max_slice(m.val_dtype) || cb.col_slice % 4) return false;
  if (it.max_row != cb.read_index[0]->max_row) return false;  // not after COMPRESSED_ROW_PADDING
  if (wl.block_num != bl.block_num) return false;             // one WLB per BLB
  for (uint64_t b = 0; b < bl.block_num; b++)
    if (bl.row_number[b] != 1) return false;
  for (uint64_t w = 0; w < wl.block_num; w++)
    if (tl.coo_block_size[w] != 1) return false;
  // every BLB inside one slice (padding repeats the last column of the piece)
  const std::vector<uint64_t> &col = cb.read_index[5]->index_arr.v;
  for (uint64_t b = 0; b < bl.block_num; b++) {
    uint64_t k0 = bl.coo_begin[b], k1 = bl.coo_begin[b + 1];
    if (k1 <= k0 || (k1 - k0) % 64) return false;
    if (col[k0] / cb.col_slice != col[k1 - 1] / cb.col_slice) return false;
  }
  return true;
}

std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  AS_CHECK(is_supported(m, sub), "format is not supported by SHARED_MEMORY_X_SLICE_TEMPLATE");
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &bl = *cb.read_index[2];
  const uint64_t S = cb.col_slice, B = bl.block_num;
  auto t = std::make_unique<Template>();
  init_template_common(*t, SHARED_MEMORY_X_SLICE_TEMPLATE, m, sub);
  t->is_atom_add = true;
  t->scalar["col_slice"] = S;
  const std::vector<uint64_t> &pcol = cb.read_index[5]->index_arr.v;
  const ValVec &pval = *cb.padding_val;

  // BLBs regrouped by slice (stable: row order kept inside a slice)
  std::vector<uint64_t> slice_of(B), order(B);
  uint64_t n_slice = 0;
  for (uint64_t b = 0; b < B; b++) {
    slice_of[b] = pcol[bl.coo_begin[b]] / S;
    n_slice = std::max(n_slice, slice_of[b] + 1);
  }
  std::vector<uint64_t> slice_begin(n_slice + 1, 0);
  for (uint64_t b = 0; b < B; b++) slice_begin[slice_of[b] + 1]++;
  for (uint64_t s = 0; s < n_slice; s++) slice_begin[s + 1] += slice_begin[s];
  {
    std::vector<uint64_t> next(slice_begin.begin(), slice_begin.end() - 1);
    for (uint64_t b = 0; b < B; b++) order[next[slice_of[b]]++] = b;
  }
  std::vector<uint64_t> row(B), nz_begin(B + 1, 0);
  t->col_index_arr.assign(std::vector<uint64_t>(pcol.size()), S <= 65536 ? UNSIGNED_SHORT : UNSIGNED_INT);
  t->val_arr.resize(pval.size());
  uint64_t max_nnz = 0;
  for (uint64_t i = 0; i < B; i++) {
    uint64_t b = order[i], k0 = bl.coo_begin[b], n = bl.coo_begin[b + 1] - k0, base = slice_of[b] * S;
    row[i] = bl.first_row[b];
    nz_begin[i + 1] = nz_begin[i] + n;
    max_nnz = std::max(max_nnz, n);
    for (uint64_t k = 0; k < n; k++) {
      AS_CHECK(pcol[k0 + k] >= base && pcol[k0 + k] - base < S, "element outside the slice of its BLB");
      t->col_index_arr.v[nz_begin[i] + k] = pcol[k0 + k] - base;
      t->val_arr[nz_begin[i] + k] = pval[k0 + k];
    }
  }
  t->global_sort_index = apply_global_sort(m, sub, row, B);
  t->scalar["max_BLB_nnz"] = max_nnz;

  // work groups: the BLBs of a slice are cut into runs of about `target` elements, one workgroup
  // trip (one copy of the slice into LDS) each
  uint64_t total = nz_begin[B];
  uint64_t target = std::max<uint64_t>(4 * S, std::min<uint64_t>(16 * S, total / 512 + 1));
  std::vector<uint64_t> group_first_block, group_slice;
  for (uint64_t s = 0; s < n_slice; s++) {
    uint64_t b0 = slice_begin[s], b1 = slice_begin[s + 1];
    if (b0 == b1) continue;
    uint64_t slice_nnz = nz_begin[b1] - nz_begin[b0];
    uint64_t parts = std::max<uint64_t>(1, (slice_nnz + target / 2) / target);
    uint64_t per = (slice_nnz + parts - 1) / parts, cur = b0;
    while (cur < b1) {
      group_first_block.push_back(cur);
      group_slice.push_back(s);
      uint64_t end = cur, lim = nz_begin[cur] + per;
      while (end < b1 && (end == cur || nz_begin[end + 1] <= lim)) end++;
      cur = end;
    }
  }
  group_first_block.push_back(B);
  t->scalar["group_num"] = group_slice.size();

  auto add = [&](const char *name, std::vector<uint64_t> v, DType dt) {
    TArr a;
    a.name = name;
    a.a.assign(std::move(v), dt);
    t->arrays.push_back(std::move(a));
  };
  uint64_t mx = *std::max_element(row.begin(), row.end());
  std::vector<uint64_t> unit_row, group_first_unit;
  unit_row.reserve(total / 64);
  for (uint64_t i = 0; i < B; i++) unit_row.insert(unit_row.end(), (nz_begin[i + 1] - nz_begin[i]) / 64, row[i]);
  for (uint64_t b : group_first_block) group_first_unit.push_back(nz_begin[b] / 64);
  add("row_index_of_unit", std::move(unit_row), suitable_dtype(mx));
  add("group_first_unit", std::move(group_first_unit), suitable_dtype(total / 64));
  add("group_slice", std::move(group_slice), suitable_dtype(n_slice));
  // the BLB view of the same layout, kept on the host for inspection only
  add("row_index_of_block_level_block", std::move(row), suitable_dtype(mx));
  add("block_nz_begin_offset", std::move(nz_begin), suitable_dtype(total));
  add("group_first_block", std::move(group_first_block), suitable_dtype(B));
  for (const char *host_only : {"row_index_of_block_level_block", "block_nz_begin_offset", "group_first_block"})
    t->find(host_only)->on_device = false;
  tpl_shared_memory_x_slice::set_default_launch(*t);
  return t;
}

void try_all_compress(Template &t) {
  TArr &g = *t.find("group_first_unit");
  if (!g.c.active()) init_linear_compressor(g.a, g.c, true);
  TArr &s = *t.find("group_slice");
  if (!s.c.active() && !init_linear_compressor(s.a, s.c, true)) init_cycle_increase_compressor(s.a, s.c, true);
}

void set_default_launch(Template &t) {
  if (t.thread_num_in_block == 0) t.thread_num_in_block = 1024;
  t.tblock_num = std::max<uint64_t>(1, std::min<uint64_t>(t.sc("group_num"), (1ull << 31) - 1));
  t.dynamic_lds_bytes = t.sc("col_slice") * (uint64_t)dtype_size(t.val_dtype);
}

std::string kernel_source(const Template &t) {
  const std::string vt = value_type_name(t), ct = dtype_c_name(t.col_index_arr.dt);
  AS_CHECK(t.val_arr.size() < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
  AS_CHECK(t.thread_num_in_block % 64 == 0 && t.thread_num_in_block >= 64 && t.thread_num_in_block <= 1024,
           "thread_num_in_block must be a multiple of 64 up to 1024");
  const uint64_t S = t.sc("col_slice"), G = t.sc("group_num");
  const std::string id = std::to_string(t.sub), B = std::to_string(t.thread_num_in_block), Ss = std::to_string(S) + "u";
  // x is read from kernal_first_col_index on; columns of the sub-matrix are relative to it
  const uint64_t x_len = t.matrix_cols - t.kernal_first_col_index;
  std::string s;
  s += "extern \"C\" __global__ void __launch_bounds__(" + B + ") spmv_" + id + "(" + kernel_signature(t) + ")\n{\n";
  s += "  typedef " + vt + " val4_t __attribute__((ext_vector_type(4)));\n";
  s += "  typedef " + ct + " col4_t __attribute__((ext_vector_type(4)));\n";
  s += "  extern __shared__ __attribute__((aligned(16))) unsigned char as_dynamic_lds[];\n";
  s += "  " + vt + " *x_slice = (" + vt + " *)as_dynamic_lds;\n";
  s += "  const unsigned int lane = threadIdx.x & 63u, wave_in_block = threadIdx.x >> 6, wave_num = " + B + "u >> 6;\n";
  s += "  const " + vt + " *x_sub = device_x_arr + " + std::to_string(t.kernal_first_col_index) + "u;\n";
  s += "  for (unsigned int grp = as_xcd_block_index(); grp < " + std::to_string(G) + "u; grp += gridDim.x)\n  {\n";
  s += "    unsigned int next_grp = grp + 1u, slice, first_unit, next_first_unit;\n";
  s += "    " + code_of_meta_read(t, "group_slice", "slice", "grp");
  s += "    " + code_of_meta_read(t, "group_first_unit", "first_unit", "grp");
  s += "    " + code_of_meta_read(t, "group_first_unit", "next_first_unit", "next_grp");
  s += "    const unsigned int col0 = slice * " + Ss + ";\n";
  s += "    const unsigned int slice_len = min(" + Ss + ", " + std::to_string(x_len) + "u - col0);\n";
  s += "    as_barrier();\n";   // readers of the previous slice are done
  // full slices are copied with a fixed trip count so that all loads of a lane are in flight together
  const uint64_t copy_trips = (S + 4 * t.thread_num_in_block - 1) / (4 * t.thread_num_in_block);
  s += "    if (slice_len == " + Ss + ")\n    {\n";
  s += "      val4_t stage[" + std::to_string(copy_trips) + "];\n";
  s += "      #pragma unroll\n      for (unsigned int k = 0; k < " + std::to_string(copy_trips) + "u; k++)\n";
  s += "      {\n        const unsigned int i = (k * " + B + "u + threadIdx.x) * 4u;\n";
  s += "        if (i < " + Ss + ") stage[k] = *(const val4_t *)(x_sub + col0 + i);\n      }\n";
  s += "      #pragma unroll\n      for (unsigned int k = 0; k < " + std::to_string(copy_trips) + "u; k++)\n";
  s += "      {\n        const unsigned int i = (k * " + B + "u + threadIdx.x) * 4u;\n";
  s += "        if (i < " + Ss + ") *(val4_t *)(x_slice + i) = stage[k];\n      }\n";
  s += "    }\n    else\n    {\n";
  s += "      for (unsigned int i = threadIdx.x * 4u; i + 4u <= slice_len; i += " + B + "u * 4u)\n";
  s += "        *(val4_t *)(x_slice + i) = *(const val4_t *)(x_sub + col0 + i);\n";
  s += "      if (threadIdx.x < (slice_len & 3u)) x_slice[(slice_len & ~3u) + threadIdx.x] = x_sub[col0 + (slice_len & ~3u) + threadIdx.x];\n";
  s += "    }\n";
  s += "    as_barrier();\n";
  // K steps of 4 units per trip: all loads of the K steps are issued before the first use
  const std::string Ks = std::to_string(kBatch);
  s += "    for (unsigned int ub = first_unit + wave_in_block * 4u; ub < next_first_unit; ub += wave_num * 4u * " + Ks + "u)\n    {\n";
  s += "      const unsigned int u0 = ub + (lane >> 4);\n";
  s += "      val4_t a[" + Ks + "];\n      col4_t c[" + Ks + "];\n      unsigned int unit_row[" + Ks + "];\n";
  s += "      #pragma unroll\n      for (unsigned int k = 0; k < " + Ks + "u; k++)\n      {\n";
  s += "        const unsigned int u = u0 + k * wave_num * 4u;\n";
  s += "        a[k] = 0; c[k] = 0; unit_row[k] = 0;\n";
  s += "        if (u < next_first_unit)\n        {\n";
  s += "          const unsigned int nz = u * 64u + (lane & 15u) * 4u;\n";
  s += "          a[k] = as_ldnt((const val4_t *)(val_arr + nz));\n";
  s += "          c[k] = as_ldnt((const col4_t *)(col_index_arr + nz));\n";
  s += "          " + code_of_meta_read(t, "row_index_of_unit", "unit_row[k]", "u");
  s += "        }\n      }\n";
  s += "      #pragma unroll\n      for (unsigned int k = 0; k < " + Ks + "u; k++)\n      {\n";
  s += "        const unsigned int u = u0 + k * wave_num * 4u;\n";
  s += "        " + vt + " acc = 0;\n";
  s += "        #pragma unroll\n        for (int j = 0; j < 4; j++) acc += a[k][j] * x_slice[(unsigned int)c[k][j]];\n";
  s += "        acc = as_group_sum<16>(acc);\n";
  s += "        if (u < next_first_unit && (lane & 15u) == 15u)\n";
  s += "          as_atomic_add(device_y_arr + unit_row[k]" +
       (!t.global_sort_index && t.kernal_first_row_index != 0 ? " + " + std::to_string(t.kernal_first_row_index) + "u" : std::string()) +
       ", acc);\n";
  s += "      }\n    }\n  }\n}\n";
  return s;
}

}  // namespace tpl_shared_memory_x_slice
}  // namespace asx
