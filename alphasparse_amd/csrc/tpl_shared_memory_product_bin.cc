// SHARED_MEMORY_PRODUCT_BIN_TEMPLATE (no upstream counterpart): short rows whose columns are spread
// over a vector much larger than the L2 cache.  A read of x that misses L2 moves a whole cache line
// for one value, so a kernel that walks such rows is bound by that traffic, not by its format.  This
// template never gathers from HBM; it runs two passes over the 2-D tiles of
// COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY (elements ordered by column
// slice, then row group, then row):
//
//   spmv_<sub>         slice by slice: a workgroup copies its slice of x into LDS, multiplies every
//                      element of its trip by its x value (LDS read) and writes the product to the
//                      place the element has in row-group order (a stored 32-bit position; the
//                      elements of a (slice, row group) bin stay together, so the writes come in runs);
//   spmv_<sub>_finish  summing group by summing group (consecutive rows of one row group, as many as
//                      fit a small number of LDS slots: rows x longest row of the group): one workgroup
//                      owns the group, streams its products (contiguous) with 128-bit loads and drops
//                      each into its own LDS slot (j-th element of row r -> slot j * rows + r: plain LDS
//                      stores, no atomics, LDS atomics retire about one lane per clock); then one lane
//                      per row adds the row's slots up and stores the row to y (nobody else writes it).
//                      The groups are small so that several workgroups share a CU and hide each
//                      other's dependent phases (table reads, stream, barrier, row sums, y index).
//
// Per element: value + 16-bit column inside the slice + 32-bit position (first pass), 16-bit LDS slot
// (second pass), and the product written once and read once.  No access to HBM is a gather.
// The slots of a summing group cover rows x longest row: the format is for short rows (best sorted).
#include "templates.hpp"

namespace asx {
namespace tpl_shared_memory_product_bin {

static const uint64_t kLdsBytes = 163840;   // LDS of one CU
static const uint64_t kCuNum = 256;
static const uint64_t kUnit = 256;          // elements of one wavefront step of the first pass (64 lanes x 4)
static const unsigned kBatch = 2;           // wavefront steps whose loads are in flight together
static const uint64_t kBand = 4096;         // rows of y whose rows of the strip are summed and stored together
// Rows of a lane whose place in y is read ahead in the second pass: as many as a lane has in the summing group of
// an average row (`typical_group_rows`: the groups' sizes averaged over the rows), between 4 and 8.  Rows beyond them read their place between the stores of the rows before, one round trip
// each (C5, 5-16 rows per lane: second pass 43.6 us with 4, 40.2 with 8, 44.3 with 12, 45.9 with 16 -- the loads
// are issued for every lane whether its group has that many rows or not, and skipping them by a test on the
// group's size cost more than it saved, 45.0; C3, 2.6 rows per lane: 15.7 us with 2 or 4, 16.1 with 9).
static unsigned y_prefetch(const Template &t) {
  const uint64_t per_lane = (t.sc("typical_group_rows") + t.finish_thread_num - 1) / std::max<uint64_t>(1, t.finish_thread_num);
  return (unsigned)std::min<uint64_t>(8, std::max<uint64_t>(4, per_lane));
}
static const uint64_t kShortRow = 4;        // longest row that is taken band by band

bool is_supported(const Matrix &m, uint64_t sub) {
  const DenseItem &it = m.items[sub];
  const CompressedBlock &cb = *it.cb;
  const uint64_t S = cb.col_slice, R = cb.row_group, vs = (uint64_t)dtype_size(m.val_dtype);
  if (S == 0 || R == 0 || S > 65536 || R > 65536 || S % 4 || S * vs > kLdsBytes) return false;
  if (it.max_row != cb.read_index[0]->max_row) return false;  // not after COMPRESSED_ROW_PADDING
  if (sub_block_is_col_restricted(m, sub)) return false;      // the second pass stores whole rows
  const Index &bl = *cb.read_index[2];
  const std::vector<uint64_t> &row = cb.read_index[0]->index_arr.v, &col = cb.read_index[1]->index_arr.v;
  if (bl.block_num == 0 || bl.coo_begin[bl.block_num] != row.size()) return false;
  for (uint64_t b = 0; b < bl.block_num; b++) {
    uint64_t k0 = bl.coo_begin[b], k1 = bl.coo_begin[b + 1];
    if (k1 <= k0) return false;
    for (uint64_t k = k0 + 1; k < k1; k++)
      if (col[k] / S != col[k0] / S || row[k] / R != row[k0] / R || row[k] < row[k - 1]) return false;
  }
  // every row must fit its slots (+ 1 spare) into LDS and into 16-bit slot numbers
  std::vector<uint64_t> len(it.max_row - it.min_row + 1, 0);
  for (uint64_t r : row) len[r]++;
  const uint64_t longest = len.empty() ? 0 : *std::max_element(len.begin(), len.end());
  return longest + 1 <= 65536 && (longest + 1) * vs <= kLdsBytes;
}

// Slot budget of a summing group.  The products of a (slice, row group) bin are written in one run per summing
// group of the row group, and short runs cost write bandwidth: the budget grows with the number of slices so
// that an average run keeps about 16 products.  At least 2048 slots, at most 64 KB of LDS, and never less than
// the longest row needs.
static uint64_t slot_budget(uint64_t slices, uint64_t longest_row, uint64_t vs) {
  const uint64_t cap = std::min<uint64_t>(std::max<uint64_t>(2048, 16 * slices), 65536 / vs);
  return std::max(cap, longest_row + 1);
}

// Rows [r0, r1) cut into groups of consecutive rows whose slots (rows x longest row, + 1 spare) fit `cap`:
// appends the first row and the width of every group and returns how many there are.
static uint64_t cut_rows(const std::vector<uint64_t> &len, uint64_t r0, uint64_t r1, uint64_t cap,
                         std::vector<uint64_t> *first_row, std::vector<uint64_t> *width) {
  uint64_t groups = 0;
  for (uint64_t r = r0; r < r1; groups++) {
    const uint64_t start = r;
    uint64_t w = 0;
    while (r < r1) {
      const uint64_t w2 = std::max(w, len[r]);
      if (r > start && (r - start + 1) * w2 + 1 > cap) break;
      w = w2;
      r++;
    }
    if (first_row) {
      first_row->push_back(start);
      width->push_back(w);
    }
  }
  return groups;
}

std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  AS_CHECK(is_supported(m, sub), "format is not supported by SHARED_MEMORY_PRODUCT_BIN_TEMPLATE");
  const DenseItem &it = m.items[sub];
  const CompressedBlock &cb = *it.cb;
  const uint64_t S = cb.col_slice, R = cb.row_group, vs = (uint64_t)dtype_size(m.val_dtype);
  const std::vector<uint64_t> &row = cb.read_index[0]->index_arr.v, &col = cb.read_index[1]->index_arr.v;
  const ValVec &val = *cb.val;
  const uint64_t n = row.size(), sub_rows = it.max_row - it.min_row + 1, sub_cols = it.max_col - it.min_col + 1;
  const uint64_t nsl = (sub_cols + S - 1) / S, nrg = (sub_rows + R - 1) / R;
  auto t = std::make_unique<Template>();
  init_template_common(*t, SHARED_MEMORY_PRODUCT_BIN_TEMPLATE, m, sub);
  t->is_atom_add = false;
  t->scalar["col_slice"] = S;
  t->scalar["row_group"] = R;
  t->scalar["sub_rows"] = sub_rows;
  t->scalar["slice_num"] = nsl;

  // y row of every row of the sub-matrix (through the sort permutation when there is one)
  std::vector<uint64_t> y_row(sub_rows);
  for (uint64_t r = 0; r < sub_rows; r++) y_row[r] = r;
  t->global_sort_index = apply_global_sort(m, sub, y_row, sub_rows);

  // Row order of the template.  Under a sort the rows of equal length are neighbours but their places in y
  // are far apart, and the second pass would write y a few bytes per line at a time.  The template
  // therefore takes the rows of up to kShortRow elements (the bulk of such a strip) band by band of y (kBand
  // rows of y each) and only inside a band by length (longest first): all rows of a band are stored at about
  // the same time and their lines of y leave the cache whole.  Longer rows stay in front in sorted order:
  // mixed into the bands they would leave most slots of their summing groups empty.  Without a sort the
  // order is the matrix's.
  std::vector<uint64_t> len(sub_rows, 0), new_of_old(sub_rows);
  for (uint64_t k = 0; k < n; k++) len[row[k]]++;
  {
    std::vector<uint64_t> by_band(sub_rows);
    for (uint64_t r = 0; r < sub_rows; r++) by_band[r] = r;
    if (t->global_sort_index)
      std::sort(by_band.begin(), by_band.end(), [&](uint64_t a, uint64_t b) {
        const uint64_t ba = len[a] > kShortRow ? 0 : 1 + y_row[a] / kBand, bb = len[b] > kShortRow ? 0 : 1 + y_row[b] / kBand;
        if (ba != bb) return ba < bb;
        if (len[a] != len[b]) return len[a] > len[b];
        return y_row[a] < y_row[b];
      });
    std::vector<uint64_t> len_new(sub_rows), y_new(sub_rows);
    for (uint64_t i = 0; i < sub_rows; i++) {
      new_of_old[by_band[i]] = i;
      len_new[i] = len[by_band[i]];
      y_new[i] = y_row[by_band[i]];
    }
    len.swap(len_new);
    y_row.swap(y_new);
  }
  // elements by (slice, row in template order): two stable counting sorts
  std::vector<uint32_t> order(n);
  {
    std::vector<uint64_t> first(std::max(sub_rows, nsl) + 1, 0);
    std::vector<uint32_t> by_row(n);
    for (uint64_t k = 0; k < n; k++) first[new_of_old[row[k]] + 1]++;
    for (uint64_t r = 0; r < sub_rows; r++) first[r + 1] += first[r];
    for (uint64_t k = 0; k < n; k++) by_row[first[new_of_old[row[k]]]++] = (uint32_t)k;
    std::fill(first.begin(), first.end(), 0);
    for (uint64_t k = 0; k < n; k++) first[col[k] / S + 1]++;
    for (uint64_t q = 0; q < nsl; q++) first[q + 1] += first[q];
    for (uint64_t i = 0; i < n; i++) order[first[col[by_row[i]] / S]++] = by_row[i];
  }

  // first-pass arrays slice by slice, every slice padded to whole units; bins = (row group, slice) pieces
  // of that stream
  std::vector<uint64_t> lcol, bin_begin(nrg * nsl, 0), bin_size(nrg * nsl, 0), slice_first_unit(nsl + 1, 0);
  std::vector<uint64_t> elem_row;  // row inside the group of every first-pass element
  lcol.reserve(n + nsl * kUnit);
  elem_row.reserve(n + nsl * kUnit);
  t->val_arr.reserve(n + nsl * kUnit);
  uint64_t cur_slice = 0;
  auto close_slices_up_to = [&](uint64_t s) {  // pad the open slice, give empty slices an empty unit range
    while (cur_slice < s) {
      while (lcol.size() % kUnit) {
        lcol.push_back(0);
        elem_row.push_back(0);
        t->val_arr.push_back(0.0);
      }
      slice_first_unit[++cur_slice] = lcol.size() / kUnit;
    }
  };
  for (uint64_t i = 0; i < n; i++) {
    const uint64_t k = order[i], s = col[k] / S, r = new_of_old[row[k]], g = r / R;
    close_slices_up_to(s);
    uint64_t &bb = bin_begin[g * nsl + s], &bs = bin_size[g * nsl + s];
    if (bs == 0) bb = lcol.size();
    bs++;
    lcol.push_back(col[k] - s * S);
    elem_row.push_back(r - g * R);
    t->val_arr.push_back(val[k]);
  }
  close_slices_up_to(nsl);
  const uint64_t padded = lcol.size();
  AS_CHECK(padded < (1ull << 32), "sub-matrix too large for 32-bit element offsets");

  // Summing groups: consecutive rows of one row group whose slots (rows x longest row, + 1 spare) fit
  // the budget.
  const uint64_t longest = *std::max_element(len.begin(), len.end()), cap = slot_budget(nsl, longest, vs);
  std::vector<uint64_t> sum_first_row, sum_width, sum_of_row(sub_rows);
  for (uint64_t r0 = 0; r0 < sub_rows;) {
    // a piece of one row group and one band of y (or of the long rows in front)
    uint64_t r1 = std::min(sub_rows, (r0 / R + 1) * R);
    if (t->global_sort_index)
      for (uint64_t r = r0 + 1; r < r1; r++)
        if (len[r0] > kShortRow ? len[r] <= kShortRow : y_row[r] / kBand != y_row[r0] / kBand) { r1 = r; break; }
    // as many groups as the budget asks for, but of about equal size: the smallest budget that gives that many
    const uint64_t groups = cut_rows(len, r0, r1, cap, nullptr, nullptr);
    uint64_t lo = longest + 1, hi = cap;
    while (lo < hi) {
      const uint64_t mid = (lo + hi) / 2;
      if (cut_rows(len, r0, r1, mid, nullptr, nullptr) <= groups) hi = mid; else lo = mid + 1;
    }
    cut_rows(len, r0, r1, lo, &sum_first_row, &sum_width);
    r0 = r1;
  }
  for (uint64_t q = 0; q < sum_first_row.size(); q++) {
    const uint64_t end = q + 1 < sum_first_row.size() ? sum_first_row[q + 1] : sub_rows;
    for (uint64_t r = sum_first_row[q]; r < end; r++) sum_of_row[r] = q;
  }
  const uint64_t nsum = sum_first_row.size();
  sum_first_row.push_back(sub_rows);
  // Second-pass order: summing group by summing group (so row group by row group), inside a group in the
  // order of the first pass (slice by slice), every group padded to whole units.  The padding is never
  // written: it keeps the zeros of the upload.  Slot of an element in the LDS of its group:
  // (its rank inside its row) * rows + (row inside the group); padding goes to the spare slot rows * width.
  std::vector<uint64_t> sum_first_unit(nsum + 1, 0), fill(nsum, 0);
  for (uint64_t g = 0; g < nrg; g++)
    for (uint64_t s = 0; s < nsl; s++)
      for (uint64_t o = 0; o < bin_size[g * nsl + s]; o++)
        fill[sum_of_row[g * R + elem_row[bin_begin[g * nsl + s] + o]]]++;
  uint64_t max_slots = 1;
  for (uint64_t q = 0; q < nsum; q++) {
    sum_first_unit[q + 1] = sum_first_unit[q] + (fill[q] + kUnit - 1) / kUnit;
    max_slots = std::max(max_slots, (sum_first_row[q + 1] - sum_first_row[q]) * sum_width[q] + 1);
  }
  const uint64_t product_len_units = sum_first_unit[nsum];
  std::vector<uint64_t> dest(padded, 0), slot(product_len_units * kUnit), seen(sub_rows, 0);
  for (uint64_t q = 0; q < nsum; q++) {
    std::fill(slot.begin() + sum_first_unit[q] * kUnit, slot.begin() + sum_first_unit[q + 1] * kUnit,
              (sum_first_row[q + 1] - sum_first_row[q]) * sum_width[q]);
    fill[q] = sum_first_unit[q] * kUnit;
  }
  for (uint64_t g = 0; g < nrg; g++)
    for (uint64_t s = 0; s < nsl; s++)
      for (uint64_t o = 0; o < bin_size[g * nsl + s]; o++) {
        const uint64_t k = bin_begin[g * nsl + s] + o, r = g * R + elem_row[k], q = sum_of_row[r];
        dest[k] = fill[q];
        slot[fill[q]++] = seen[r]++ * (sum_first_row[q + 1] - sum_first_row[q]) + (r - sum_first_row[q]);
      }
  AS_CHECK(max_slots <= 65536 && max_slots * vs <= kLdsBytes, "a row group does not fit its LDS slots");
  t->scalar["max_slots"] = max_slots;
  t->scalar["sum_group_num"] = nsum;
  {
    uint64_t squares = 0;
    for (uint64_t q = 0; q < nsum; q++) squares += (sum_first_row[q + 1] - sum_first_row[q]) * (sum_first_row[q + 1] - sum_first_row[q]);
    t->scalar["typical_group_rows"] = squares / std::max<uint64_t>(1, sub_rows);
  }
  const uint64_t product_len = slot.size();
  AS_CHECK(product_len < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
  // first-pass padding goes to a spare slot behind the products
  {
    std::vector<bool> real(padded, false);
    for (uint64_t i = 0; i < nrg * nsl; i++)
      for (uint64_t o = 0; o < bin_size[i]; o++) real[bin_begin[i] + o] = true;
    for (uint64_t k = 0; k < padded; k++)
      if (!real[k]) dest[k] = product_len;
  }
  t->col_index_arr.assign(std::move(lcol), UNSIGNED_SHORT);
  t->scratch_bytes = (product_len + 1) * vs;
  t->scalar["product_len"] = product_len;

  // first pass: trips of about equal cost (units of elements + one slice copy each), cut inside slices
  const uint64_t unit_bytes = kUnit * (2 * vs + 6), slice_units = (S * vs + unit_bytes - 1) / unit_bytes;
  const uint64_t total_units = padded / kUnit;
  uint64_t want = kCuNum * std::max<uint64_t>(1, kLdsBytes / (S * vs));
  want = std::max<uint64_t>(1, std::min<uint64_t>(want, (total_units + 63) / 64));
  uint64_t nonempty = 0;
  for (uint64_t s = 0; s < nsl; s++) nonempty += slice_first_unit[s + 1] > slice_first_unit[s];
  const uint64_t per_trip = (total_units + (nonempty + want) * slice_units) / want + 1;
  std::vector<uint64_t> group_slice, group_first_unit;
  for (uint64_t s = 0; s < nsl; s++) {
    uint64_t u0 = slice_first_unit[s], u1 = slice_first_unit[s + 1];
    if (u1 == u0) continue;
    uint64_t room = per_trip > slice_units ? per_trip - slice_units : 1;
    uint64_t parts = std::max<uint64_t>(1, (u1 - u0 + room / 2) / room), per = (u1 - u0 + parts - 1) / parts;
    for (uint64_t u = u0; u < u1; u += per) {
      group_slice.push_back(s);
      group_first_unit.push_back(u);
    }
  }
  // a trip ends where the next one starts; the last one at the end of its slice, which is where the
  // next non-empty slice starts
  group_first_unit.push_back(total_units);
  t->scalar["group_num"] = group_slice.size();

  auto add = [&](const char *name, std::vector<uint64_t> v, DType at_least) {
    TArr a;
    a.name = name;
    uint64_t mx = v.empty() ? 0 : *std::max_element(v.begin(), v.end());
    a.a.assign(std::move(v), IArr::at_least(at_least, mx));
    t->arrays.push_back(std::move(a));
  };
  add("group_slice", std::move(group_slice), UNSIGNED_CHAR);
  add("group_first_unit", std::move(group_first_unit), UNSIGNED_CHAR);
  add("product_position", std::move(dest), UNSIGNED_INT);
  // read with scalar loads, which need 32-bit entries
  add("sum_group_first_row", std::move(sum_first_row), UNSIGNED_INT);
  add("sum_group_first_unit", std::move(sum_first_unit), UNSIGNED_INT);
  add("sum_group_width", std::move(sum_width), UNSIGNED_INT);
  add("slot_in_group", std::move(slot), UNSIGNED_SHORT);
  add("y_row_index", std::move(y_row), UNSIGNED_CHAR);
  tpl_shared_memory_product_bin::set_default_launch(*t);
  return t;
}

void try_all_compress(Template &t) {
  for (const char *name : {"group_first_unit", "sum_group_first_unit", "sum_group_first_row", "y_row_index"}) {
    TArr &a = *t.find(name);
    if (!a.c.active()) init_linear_compressor(a.a, a.c, true);
  }
  TArr &s = *t.find("group_slice");
  if (!s.c.active() && !init_linear_compressor(s.a, s.c, true)) init_cycle_increase_compressor(s.a, s.c, true);
  TArr &w = *t.find("sum_group_width");
  if (!w.c.active() && !init_constant_compressor(w.a, w.c, true) && w.a.size() > 2) init_branch_compressor(w.a, w.c, 5);
}

void set_default_launch(Template &t) {
  const uint64_t vs = (uint64_t)dtype_size(t.val_dtype);
  if (t.thread_num_in_block == 0) t.thread_num_in_block = 1024;
  t.tblock_num = std::max<uint64_t>(1, std::min<uint64_t>(t.sc("group_num"), (1ull << 31) - 1));
  t.dynamic_lds_bytes = t.sc("col_slice") * vs;
  t.finish_tblock_num = std::max<uint64_t>(1, std::min<uint64_t>(t.sc("sum_group_num"), (1ull << 31) - 1));
  // a lane for every eighth slot of the largest group, between 256 and 512: several workgroups share a CU
  t.finish_thread_num = std::min<uint64_t>(512, std::max<uint64_t>(256, t.sc("max_slots") / 8 / 64 * 64));
  t.finish_lds_bytes = t.sc("max_slots") * vs;
}

std::string kernel_source(const Template &t) {
  const std::string vt = value_type_name(t);
  AS_CHECK(t.col_index_arr.dt == UNSIGNED_SHORT && t.arr("slot_in_group").a.dt == UNSIGNED_SHORT &&
               t.arr("product_position").a.dt == UNSIGNED_INT, "slice columns and LDS slots must be 16 bits wide, positions 32");
  AS_CHECK(t.thread_num_in_block % 64 == 0 && t.thread_num_in_block >= 64 && t.thread_num_in_block <= 1024,
           "thread_num_in_block must be a multiple of 64 up to 1024");
  const uint64_t S = t.sc("col_slice"), R = t.sc("row_group"), G = t.sc("group_num"), rows = t.sc("sub_rows");
  const uint64_t nsum = t.sc("sum_group_num");
  const std::string id = std::to_string(t.sub), B = std::to_string(t.thread_num_in_block) + "u";
  const std::string Ss = std::to_string(S) + "u", Rs = std::to_string(R) + "u", Ks = std::to_string(kBatch);
  const std::string FB = std::to_string(t.finish_thread_num);
  const uint64_t x_len = t.matrix_cols - t.kernal_first_col_index;
  const bool wide_copy = t.kernal_first_col_index % 4 == 0;
  std::string s;
  // ---- first pass: products -------------------------------------------------------------------
  s += "extern \"C\" __global__ void __launch_bounds__(" + std::to_string(t.thread_num_in_block) + ") spmv_" + id + "(" +
       kernel_signature(t) + carried_finish_signature(t) + ")\n{\n";
  s += carried_finish_prologue(t, t.thread_num_in_block);
  const std::string Cs = std::to_string(16 / dtype_size(t.val_dtype));
  s += "  typedef " + vt + " val16_t __attribute__((ext_vector_type(" + Cs + ")));\n";  // 16 bytes of values
  s += "  extern __shared__ __attribute__((aligned(16))) unsigned char as_dynamic_lds[];\n";
  s += "  " + vt + " *x_slice = (" + vt + " *)as_dynamic_lds;\n";
  s += "  " + vt + " *product = (" + vt + " *)scratch_arr;\n";
  s += "  const unsigned int lane = threadIdx.x & 63u, wave_in_block = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);\n";
  s += "  const unsigned int stride = (" + B + " >> 6) * 256u;\n";
  s += "  const " + vt + " *x_sub = device_x_arr + " + std::to_string(t.kernal_first_col_index) + "u;\n";
  s += "  for (unsigned int grp = as_xcd_block_index(as_block, as_grid); grp < " + std::to_string(G) + "u; grp += as_grid)\n  {\n";
  s += "    unsigned int next_grp = grp + 1u, slice, unit_begin, unit_end;\n";
  s += "    " + code_of_meta_read(t, "group_slice", "slice", "grp");
  s += "    " + code_of_meta_read(t, "group_first_unit", "unit_begin", "grp");
  s += "    " + code_of_meta_read(t, "group_first_unit", "unit_end", "next_grp");
  s += "    const unsigned int col0 = slice * " + Ss + ";\n";
  s += "    const unsigned int slice_len = min(" + Ss + ", " + std::to_string(x_len) + "u - col0);\n";
  s += "    __syncthreads();\n";  // readers of the previous slice are done
  if (wide_copy) {
    // 16 bytes per lane and load (the 64 lanes of a load read one contiguous kilobyte); four loads of a lane
    // are requested before the first is stored
    s += "    for (unsigned int i0 = threadIdx.x * " + Cs + "u; i0 + " + Cs + "u <= slice_len; i0 += " + B + " * 4u * " + Cs + "u)\n    {\n";
    s += "      val16_t part[4];\n";
    s += "      #pragma unroll\n      for (int j = 0; j < 4; j++)\n";
    s += "        if (i0 + j * " + B + " * " + Cs + "u + " + Cs + "u <= slice_len) part[j] = *(const val16_t *)(x_sub + col0 + i0 + j * " + B + " * " + Cs + "u);\n";
    s += "      #pragma unroll\n      for (int j = 0; j < 4; j++)\n";
    s += "        if (i0 + j * " + B + " * " + Cs + "u + " + Cs + "u <= slice_len) *(val16_t *)(x_slice + i0 + j * " + B + " * " + Cs + "u) = part[j];\n";
    s += "    }\n";
    s += "    if (threadIdx.x < slice_len % " + Cs + "u) x_slice[slice_len / " + Cs + "u * " + Cs + "u + threadIdx.x] = x_sub[col0 + slice_len / " + Cs + "u * " + Cs + "u + threadIdx.x];\n";
  } else {
    s += "    for (unsigned int i = threadIdx.x; i < slice_len; i += " + B + ") x_slice[i] = x_sub[col0 + i];\n";
  }
  s += "    __syncthreads();\n";
  // Consecutive lanes take consecutive elements: the products of a run then go to consecutive places with one
  // store instruction (whole lines), instead of every fourth place with each of four.
  s += "    const unsigned int nz_end = unit_end * 256u;\n";
  s += "    for (unsigned int nz0 = unit_begin * 256u + wave_in_block * 256u; nz0 < nz_end; nz0 += stride * " + Ks + "u)\n    {\n";
  s += "      " + vt + " a[" + Ks + "][4];\n      unsigned short c[" + Ks + "][4];\n      unsigned int d[" + Ks + "][4];\n";
  s += "      #pragma unroll\n      for (int k = 0; k < " + Ks + "; k++)\n      {\n";
  s += "        if (nz0 + k * stride < nz_end)\n        {\n";
  s += "          #pragma unroll\n          for (int j = 0; j < 4; j++)\n          {\n";
  s += "            const unsigned int nz = nz0 + k * stride + j * 64u + lane;\n";
  s += "            a[k][j] = as_ldnt(val_arr + nz);\n";
  s += "            c[k][j] = as_ldnt(col_index_arr + nz);\n";
  s += "            d[k][j] = as_ldnt(product_position + nz);\n";
  s += "          }\n        }\n      }\n";
  s += "      #pragma unroll\n      for (int k = 0; k < " + Ks + "; k++)\n      {\n";
  s += "        if (nz0 + k * stride < nz_end)\n        {\n";
  s += "          #pragma unroll\n          for (int j = 0; j < 4; j++) product[d[k][j]] = a[k][j] * x_slice[(unsigned int)c[k][j]];\n";
  s += "        }\n      }\n    }\n  }\n}\n";
  // ---- second pass: row sums ------------------------------------------------------------------
  s += "extern \"C\" __global__ void __launch_bounds__(" + FB + ") spmv_" + id + "_finish(" + kernel_signature(t) + ")\n{\n";
  s += "  extern __shared__ __attribute__((aligned(16))) unsigned char as_dynamic_lds[];\n";
  s += "  " + vt + " *slots = (" + vt + " *)as_dynamic_lds;\n";
  s += "  const " + vt + " *product = (const " + vt + " *)scratch_arr;\n";
  s += "  const unsigned int lane = threadIdx.x & 63u, wave_in_block = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);\n";
  s += "  const unsigned int stride = (" + FB + "u >> 6) * 256u;\n";
  // neighbouring summing groups write neighbouring rows of y: they run on the same XCD, behind the same L2
  s += "  for (unsigned int grp = as_xcd_block_index(); grp < " + std::to_string(nsum) + "u; grp += gridDim.x)\n  {\n";
  s += "    unsigned int next_grp = grp + 1u, row0, row_end, unit_begin, unit_end, width;\n";
  s += "    " + code_of_meta_read(t, "sum_group_first_row", "row0", "grp");
  s += "    " + code_of_meta_read(t, "sum_group_first_row", "row_end", "next_grp");
  s += "    " + code_of_meta_read(t, "sum_group_first_unit", "unit_begin", "grp");
  s += "    " + code_of_meta_read(t, "sum_group_first_unit", "unit_end", "next_grp");
  s += "    " + code_of_meta_read(t, "sum_group_width", "width", "grp");
  s += "    const unsigned int live = row_end - row0;\n";
  // the places in y of the lane's first rows are requested now and used after the sums
  s += "    unsigned int y_place[" + std::to_string(y_prefetch(t)) + "];\n";
  s += "    #pragma unroll\n    for (int k = 0; k < " + std::to_string(y_prefetch(t)) + "; k++)\n    {\n";
  s += "      const unsigned int sub_row = row0 + min(threadIdx.x + k * " + FB + "u, live - 1u);\n";
  s += "      " + code_of_meta_read(t, "y_row_index", "y_place[k]", "sub_row");
  s += "    }\n";
  s += "    __syncthreads();\n";  // the previous group's rows are stored
  s += "    for (unsigned int i = threadIdx.x; i < width * live; i += " + FB + "u) slots[i] = 0;\n";
  s += "    __syncthreads();\n";
  s += "    const unsigned int nz_end = unit_end * 256u;\n";
  s += "    for (unsigned int nz0 = unit_begin * 256u + wave_in_block * 256u; nz0 < nz_end; nz0 += stride * " + Ks + "u)\n    {\n";
  // consecutive lanes take consecutive products: every load of the 64 lanes reads one contiguous stretch
  s += "      " + vt + " p[" + Ks + "][4];\n      unsigned short q[" + Ks + "][4];\n";
  s += "      #pragma unroll\n      for (int k = 0; k < " + Ks + "; k++)\n      {\n";
  s += "        if (nz0 + k * stride < nz_end)\n        {\n";
  s += "          #pragma unroll\n          for (int j = 0; j < 4; j++)\n          {\n";
  s += "            const unsigned int nz = nz0 + k * stride + j * 64u + lane;\n";
  s += "            p[k][j] = product[nz];\n";
  s += "            q[k][j] = as_ldnt(slot_in_group + nz);\n";
  s += "          }\n        }\n      }\n";
  s += "      #pragma unroll\n      for (int k = 0; k < " + Ks + "; k++)\n      {\n";
  s += "        if (nz0 + k * stride >= nz_end) continue;\n";
  s += "        #pragma unroll\n        for (int j = 0; j < 4; j++) slots[(unsigned int)q[k][j]] = p[k][j];\n";
  s += "      }\n    }\n";
  s += "    __syncthreads();\n";
  const std::string y_off = (!t.global_sort_index && t.kernal_first_row_index != 0 ? " + " + std::to_string(t.kernal_first_row_index) + "u" : std::string());
  s += "    #pragma unroll\n    for (int k = 0; k < " + std::to_string(y_prefetch(t)) + "; k++)\n    {\n";
  s += "      const unsigned int i = threadIdx.x + k * " + FB + "u;\n";
  s += "      if (i < live)\n      {\n";
  s += "        " + vt + " sum = 0;\n";
  s += "        for (unsigned int j = 0; j < width; j++) sum += slots[j * live + i];\n";
  s += "        device_y_arr[y_place[k]" + y_off + "] = sum;\n";
  s += "      }\n    }\n";
  s += "    for (unsigned int i = threadIdx.x + " + std::to_string(y_prefetch(t)) + "u * " + FB + "u; i < live; i += " + FB + "u)\n    {\n";
  s += "      " + vt + " sum = 0;\n";
  s += "      for (unsigned int j = 0; j < width; j++) sum += slots[j * live + i];\n";
  s += "      const unsigned int sub_row = row0 + i;\n";
  s += "      unsigned int global_row_index;\n";
  s += "      " + code_of_meta_read(t, "y_row_index", "global_row_index", "sub_row");
  s += "      device_y_arr[global_row_index" + y_off + "] = sum;\n";
  s += "    }\n  }\n}\n";
  return s;
}

}  // namespace tpl_shared_memory_product_bin
}  // namespace asx
