// UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE (+ _WITH_WARP_REDUCE): CSR5-like.
// The elements of the sub-matrix are cut into TLBs of a fixed size s regardless
// of row boundaries; W TLBs form a WLB handled by one wavefront.  Per TLB one
// packed word holds a row-start bitmap, the number of following TLBs without a
// row start, and the first row relative to the WLB.
//
// Format arrays follow upstream init_unaligned_warp_reduce_same_TLB_size_template
// (unaligned_warp_reduce_same_TLB_size_op.cc:5-297) and its helpers
// fill_empty_and_padding_to_align_warp (:434-512), get_sum_begin_bool_flag_of_each_thread
// (:1332), get_first_global_row_index_of_each_warp (:1391), get_tmp_result_reduce_offset_vec
// (:1419), get_first_relative_reduce_row_of_thread_level_block_vec (:1492), combine_meta_data
// (:1594).  The kernel is new: per-lane bitmap walk, wave-wide segmented scan of the
// "head" partials, one indexed shuffle to close each row, atomics only where a row can
// continue into another wavefront's WLB.
#include "templates.hpp"

namespace asx {
namespace {

int bit_num(uint64_t v) {  // get_max_bit_num_of_meta_data (:1575)
  int n = 0;
  while (v) { v >>= 1; n++; }
  return n;
}

struct Unaligned {
  std::vector<uint64_t> row, col;
  ValVec val;
  std::vector<uint64_t> flags;      // per TLB, bit (s-1-k) set iff element k starts a row
  std::vector<uint64_t> wlb_first_row, reduce_offset, first_rel_row;
  uint64_t s = 0, max_offset = 0, max_rel_row = 0;
  int bits_flag = 0, bits_off = 0, bits_row = 0;
};

bool build(const Matrix &m, uint64_t sub, Unaligned &u) {
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &ri = *cb.read_index[0], &ci = *cb.read_index[1], &tl = *cb.read_index[4];
  const unsigned W = m.wave;
  u.s = tl.coo_block_size[0];
  if (u.s == 0 || u.s > 60) return false;
  // one (col 0, val 0) element per row without elements, then pad the tail to W * s
  uint64_t last = 0;
  for (uint64_t k = 0; k < ri.length; k++) {
    uint64_t r = ri.index_arr[k];
    for (uint64_t e = (k == 0 ? 0 : last + 1); e < r; e++) {
      u.row.push_back(e); u.col.push_back(0); u.val.push_back(0.0);
    }
    u.row.push_back(r); u.col.push_back(ci.index_arr[k]); u.val.push_back((*cb.val)[k]);
    last = r;
  }
  uint64_t wlb_nnz = W * u.s;
  while (u.row.size() % wlb_nnz != 0) {
    u.row.push_back(u.row.back()); u.col.push_back(u.col.back()); u.val.push_back(0.0);
  }
  uint64_t T = u.row.size() / u.s;
  u.flags.assign(T, 0);
  for (uint64_t t = 0; t < T; t++)
    for (uint64_t k = 0; k < u.s; k++) {
      uint64_t g = t * u.s + k;
      bool start = (k == 0 && t % W == 0) || u.row[g] != u.row[g - 1];
      if (start) u.flags[t] |= 1ull << (u.s - 1 - k);
    }
  for (uint64_t w = 0; w < T / W; w++) u.wlb_first_row.push_back(u.row[w * wlb_nnz]);
  u.reduce_offset.assign(T, 0);
  uint64_t last_t = 0, run = 0;
  for (uint64_t t = 1; t < T; t++) {
    if (u.flags[t] == 0) run++;
    else {
      u.max_offset = std::max(u.max_offset, run);
      u.reduce_offset[last_t] = run;
      run = 0;
      last_t = t;
    }
  }
  u.max_offset = std::max(u.max_offset, run);
  u.reduce_offset[last_t] = run;
  u.first_rel_row.resize(T);
  for (uint64_t t = 0; t < T; t++) {
    if (u.flags[t] == 0) u.first_rel_row[t] = u.first_rel_row[t - 1];
    else {
      uint64_t k = 0;
      while (!(u.flags[t] >> (u.s - 1 - k) & 1)) k++;
      u.first_rel_row[t] = u.row[t * u.s + k] - u.wlb_first_row[t / W];
    }
    u.max_rel_row = std::max(u.max_rel_row, u.first_rel_row[t]);
  }
  u.bits_flag = (int)u.s;
  u.bits_off = std::max(1, bit_num(u.max_offset));
  u.bits_row = std::max(1, bit_num(u.max_rel_row));
  return u.bits_flag + u.bits_off + u.bits_row <= 64;
}

// is_supported_by_unaligned_warp_reduce_same_TLB_size_template (:299-418)
bool supported(const Matrix &m, uint64_t sub) {
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &ri = *cb.read_index[0], &bl = *cb.read_index[2], &wl = *cb.read_index[3], &tl = *cb.read_index[4];
  if (ri.max_row != m.items[sub].max_row) return false;  // no compressed-view row padding
  if (tl.ctype != NO_INDEX || !tl.row_number.present) return false;
  if (bl.block_num != 1 || wl.block_num != 1) return false;
  Unaligned u;
  return build(m, sub, u);
}

std::unique_ptr<Template> make(TemplateType type, const Matrix &m, uint64_t sub) {
  AS_CHECK(supported(m, sub), "format is not supported by the unaligned templates");
  const CompressedBlock &cb = *m.items[sub].cb;
  const unsigned W = m.wave;
  Unaligned u;
  build(m, sub, u);
  auto t = std::make_unique<Template>();
  init_template_common(*t, type, m, sub);
  t->is_atom_add = sub_block_is_col_restricted(m, sub);  // is_all_force_atom_add
  const uint64_t T = u.flags.size(), s = u.s;
  int total_bits = u.bits_flag + u.bits_off + u.bits_row;
  DType meta_dt = total_bits <= 8 ? UNSIGNED_CHAR : total_bits <= 16 ? UNSIGNED_SHORT : total_bits <= 32 ? UNSIGNED_INT : UNSIGNED_LONG;
  int word = dtype_size(meta_dt) * 8, empty = word - total_bits;
  t->scalar["global_thread_level_block_size"] = s;
  t->scalar["bit_num_of_thread_level_combine_meta"] = (uint64_t)word;
  t->scalar["bit_num_of_sum_begin_bit_flag"] = (uint64_t)u.bits_flag;
  t->scalar["bit_num_of_first_relative_reduce_row_of_thread_level_block"] = (uint64_t)u.bits_row;
  t->scalar["bit_num_of_tmp_result_reduce_offset_of_thread_level_block"] = (uint64_t)u.bits_off;
  t->scalar["WLB_num"] = T / W;
  std::vector<uint64_t> meta(T);
  for (uint64_t i = 0; i < T; i++) {
    uint64_t v = u.flags[i];
    v = (empty + u.bits_off) >= 64 ? 0 : v << (empty + u.bits_off);
    v |= u.reduce_offset[i];
    v <<= u.bits_row;
    v |= u.first_rel_row[i];
    meta[i] = word == 64 ? v : (v & ((1ull << word) - 1));
  }
  auto add = [&](const char *name, std::vector<uint64_t> v, DType dt, bool dev) {
    TArr a;
    a.name = name;
    a.a.assign(std::move(v), dt);
    a.on_device = dev;
    t->arrays.push_back(std::move(a));
  };
  std::vector<uint64_t> wfr = u.wlb_first_row;
  if (type == UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE) wfr.push_back(u.row.back() + 1);
  add("global_first_row_index_of_warp_level_block", std::move(wfr), cb.read_index[0]->index_arr.dt, true);
  add("combine_meta_of_thread_level_block", std::move(meta), meta_dt, true);
  add("first_relative_reduce_row_of_thread_level_block", u.first_rel_row, suitable_dtype(u.max_rel_row), false);
  add("tmp_result_reduce_offset_of_thread_level_block", u.reduce_offset, suitable_dtype(u.max_offset), false);
  if (m.sorted_row_index.present) {
    t->global_sort_index = true;
    add("row_index_before_sort", m.sorted_row_index.v, m.sorted_row_index.dt, true);
  } else if (cb.y_write_index.present) {  // rows sorted inside BLBs: the permutation is relative to the sub-matrix
    add("row_index_before_sort", cb.y_write_index.v, cb.y_write_index.dt, true);
  }
  // interleave: element k of TLB lane -> wlb * W * s + lane + k * W   (:282-291)
  t->col_index_arr.assign(std::vector<uint64_t>(u.col.size()), cb.read_index[1]->index_arr.dt);
  t->val_arr.resize(u.val.size());
  for (uint64_t g = 0; g < u.val.size(); g++) {
    uint64_t tlb = g / s, k = g % s, dst = (tlb / W) * (W * s) + tlb % W + k * W;
    t->col_index_arr.v[dst] = u.col[g];
    t->val_arr[dst] = u.val[g];
  }
  return t;
}

void compress(Template &t) {  // try_all_compress (:1787-1802)
  TArr &r = *t.find("global_first_row_index_of_warp_level_block");
  if (!r.c.active() && !init_linear_compressor(r.a, r.c, true)) init_cycle_increase_compressor(r.a, r.c, true);
}

std::string source(const Template &t, bool grid_stride) {
  AS_CHECK(t.wave == 64, "kernel is written for 64-lane wavefronts; build the format with wave = 64");
  AS_CHECK(t.val_arr.size() < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
  const std::string vt = value_type_name(t);
  const std::string id = std::to_string(t.sub), B = std::to_string(t.thread_num_in_block);
  const std::string waves = std::to_string(t.thread_num_in_block / 64);
  const std::string fc = std::to_string(t.kernal_first_col_index) + "u";
  const uint64_t s = t.sc("global_thread_level_block_size"), wlbs = t.sc("WLB_num");
  const uint64_t word = t.sc("bit_num_of_thread_level_combine_meta");
  const uint64_t bits_row = t.sc("bit_num_of_first_relative_reduce_row_of_thread_level_block");
  const uint64_t bits_off = t.sc("bit_num_of_tmp_result_reduce_offset_of_thread_level_block");
  const std::string mt = word == 64 ? "as_u64" : "as_u32";
  std::string write_row = t.global_sort_index
                              ? "row_index_before_sort[" + std::to_string(t.kernal_first_row_index) + "u + (ROW)]"
                          : t.local_sort_index
                              ? "(" + std::to_string(t.kernal_first_row_index) + "u + row_index_before_sort[(ROW)])"
                              : "(" + std::to_string(t.kernal_first_row_index) + "u + (ROW))";
  std::string S;
  S += "extern \"C\" __global__ void __launch_bounds__(" + B + ") spmv_" + id + "(" + kernel_signature(t) + ")\n{\n";
  S += "  const unsigned int lane = threadIdx.x & 63u;\n";
  if (grid_stride)
    S += "  for (unsigned int wlb = as_xcd_block_index() * " + waves + "u + (threadIdx.x >> 6); wlb < " + std::to_string(wlbs) +
         "u; wlb += gridDim.x * " + waves + "u)\n  {\n";
  else
    S += "  const unsigned int wlb = as_xcd_block_index() * " + waves + "u + (threadIdx.x >> 6);\n  if (wlb < " +
         std::to_string(wlbs) + "u)\n  {\n";
  S += "    unsigned int wlb_first_row;\n    " +
       code_of_meta_read(t, "global_first_row_index_of_warp_level_block", "wlb_first_row", "wlb");
  S += "    const " + mt + " meta = (" + mt + ")combine_meta_of_thread_level_block[wlb * 64u + lane];\n";
  S += "    const " + mt + " flags = meta >> " + std::to_string(word - s) + ";\n";
  S += "    const unsigned int reduce_offset = (unsigned int)((meta >> " + std::to_string(bits_row) + ") & " +
       std::to_string((1ull << bits_off) - 1) + "ull);\n";
  S += "    unsigned int row = wlb_first_row + (unsigned int)(meta & " + std::to_string((bits_row >= 64 ? ~0ull : (1ull << bits_row) - 1)) + "ull);\n";
  S += "    " + vt + " head = 0, cur = 0;\n    bool seen = false;\n";
  S += "    unsigned int nz = wlb * " + std::to_string(64 * s) + "u + lane;\n";
  S += "    #pragma unroll\n    for (int k = 0; k < " + std::to_string(s) + "; k++, nz += 64u)\n    {\n";
  S += "      if ((flags >> (" + std::to_string(s - 1) + " - k)) & 1)\n      {\n";
  S += "        if (seen)\n        {\n";
  // a segment that starts and ends inside this TLB; lane 0's first segment may continue a row of the previous WLB
  std::string wr = write_row;
  size_t pos;
  while ((pos = wr.find("(ROW)")) != std::string::npos) wr.replace(pos, 5, "row");
  if (t.is_atom_add) S += "          as_atomic_add(device_y_arr + " + wr + ", cur);\n";
  else {
    S += "          if (lane == 0u && head_is_wave_first) as_atomic_add(device_y_arr + " + wr + ", cur);\n";
    S += "          else device_y_arr[" + wr + "] = cur;\n";
  }
  S += "          head_is_wave_first = false;\n          row++;\n        }\n";
  S += "        else { head = cur; seen = true; }\n";
  S += "        cur = 0;\n      }\n";
  S += "      cur += as_ldnt(val_arr + nz) * device_x_arr[" + fc + " + (unsigned int)as_ldnt(col_index_arr + nz)];\n";
  S += "    }\n";
  S += "    if (!seen) head = cur;\n";
  // Segmented inclusive scan of the head partials: a segment is a run of lanes
  // without a row start closed by the next lane that has one, so the lane that
  // closes a row holds exactly the sum the opening lane is missing (no
  // subtraction of prefix sums, hence no cancellation).
  // (The same scan on DPP row shifts and row broadcasts -- as_wave_segmented_sum over a segment number made from
  // a ballot of `seen` and a bit count -- was measured and is no faster: the 5-point stencil of 2048 x 2048 points
  // with TLBs of 4 elements runs 138.0 us with this shuffle scan and 146.0 us with the DPP scan at 128 threads,
  // 147.0 against 155.9 us at 256 threads; 4096 rows of 8 elements take 4.8 us either way.  The kernel's time is
  // in the walk over the start flags and in the atomics on rows that cross a TLB, not in the scan.)
  S += "    " + vt + " scan = head;\n";
  S += "    int seg_start = (lane == 0u) || __shfl_up((int)seen, 1, 64);\n";
  S += "    #pragma unroll\n    for (int o = 1; o < 64; o <<= 1)\n    {\n      " + vt +
       " up = __shfl_up(scan, o, 64);\n      int up_start = __shfl_up(seg_start, o, 64);\n"
       "      if ((int)lane >= o && !seg_start) { scan += up; seg_start = up_start; }\n    }\n";
  S += "    unsigned int closing = lane + reduce_offset + 1u;\n";
  S += "    const bool reaches_end = closing > 63u;\n";
  S += "    if (reaches_end) closing = 63u;\n";
  S += "    " + vt + " closed = __shfl(scan, (int)closing, 64);\n";
  S += "    if (closing == lane) closed = 0;\n";
  S += "    if (seen)\n    {\n      const " + vt + " total = cur + closed;\n";
  if (t.is_atom_add) S += "      as_atomic_add(device_y_arr + " + wr + ", total);\n";
  else {
    S += "      if (reaches_end || (lane == 0u && head_is_wave_first)) as_atomic_add(device_y_arr + " + wr + ", total);\n";
    S += "      else device_y_arr[" + wr + "] = total;\n";
  }
  S += "    }\n  }\n}\n";
  // declare the flag used above right after the scalar declarations
  std::string decl = "    bool seen = false;\n";
  S.replace(S.find(decl), decl.size(), decl + "    bool head_is_wave_first = true;\n");
  return S;
}

}  // namespace

namespace tpl_unaligned_warp_reduce {
bool is_supported(const Matrix &m, uint64_t sub) { return supported(m, sub); }
std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  auto t = make(UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE, m, sub);
  tpl_unaligned_warp_reduce::set_default_launch(*t);
  return t;
}
void try_all_compress(Template &t) { compress(t); }
void set_default_launch(Template &t) {
  if (t.thread_num_in_block == 0) t.thread_num_in_block = 256;
  uint64_t waves = t.thread_num_in_block / 64;
  t.tblock_num = std::max<uint64_t>(1, std::min<uint64_t>((t.sc("WLB_num") + waves - 1) / waves, 256 * 32));
}
std::string kernel_source(const Template &t) { return source(t, true); }
}  // namespace tpl_unaligned_warp_reduce

namespace tpl_unaligned_warp_reduce_with_warp_reduce {
bool is_supported(const Matrix &m, uint64_t sub) { return supported(m, sub); }
std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  auto t = make(UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE, m, sub);
  tpl_unaligned_warp_reduce_with_warp_reduce::set_default_launch(*t);
  return t;
}
void try_all_compress(Template &t) { compress(t); }
// one wavefront per WLB: the grid follows from the block size (upstream :1719-1885)
void set_default_launch(Template &t) {
  if (t.thread_num_in_block == 0) t.thread_num_in_block = 256;
  uint64_t waves = t.thread_num_in_block / 64;
  t.tblock_num = std::max<uint64_t>(1, (t.sc("WLB_num") + waves - 1) / waves);
}
std::string kernel_source(const Template &t) { return source(t, false); }
}  // namespace tpl_unaligned_warp_reduce_with_warp_reduce

}  // namespace asx
