// SHARED_MEMORY_PRODUCT_BIN_TEMPLATE (no upstream counterpart): short rows whose columns are spread
// over a vector much larger than the L2 cache.  A read of x that misses L2 moves a whole cache line
// for one value, so a kernel that walks such rows is bound by that traffic, not by its format.  This
// template never gathers from HBM; it runs two passes over the elements of
// COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY, which it orders itself: by column
// slice, inside a slice by band of y (`row_group` consecutive rows of y, fewer where a band's elements
// would not fit the LDS budget), inside a band by row, the rows of a band from the longest to the
// shortest (their rank):
//
//   spmv_<sub>         slice by slice: a workgroup copies its slice of x into LDS, multiplies every
//                      element of its trip by its x value (LDS read) and writes the product to the
//                      place the element has in band order: the element's own number plus the shift of
//                      its bin (the elements of one band in one slice; they stay together, so the
//                      writes come in runs).  The top bit of the 16-bit column marks the first element
//                      of a bin; a lane finds its bin by counting the marks in front of its element
//                      (a table gives the count at the start of every 256 elements, a ballot and a bit
//                      count the rest), the shifts of the trip's bins wait in LDS beside the slice;
//   spmv_<sub>_finish  band by band: one workgroup owns the band, streams its products (contiguous)
//                      and drops each into its own LDS slot -- the j-th element of the row of rank r
//                      goes to slot first[j] + r, where first[j] counts the slots of the elements
//                      0..j-1 of all rows (a jagged-diagonal layout: no empty slots, whatever the mix
//                      of row lengths; plain LDS stores, no atomics); then one lane per rank adds its
//                      row's slots up (the lanes of a wavefront hold rows of about equal length) and
//                      leaves the sum in the row's first slot; then one lane per row of y of the band
//                      looks up the rank of its row (16 bits; 0xffff = the row belongs to another
//                      strip) and stores the sum: consecutive lanes, consecutive rows of y.
//                      Bands are small enough for several workgroups to share a CU and hide each
//                      other's dependent phases (table reads, stream, barrier, row sums, stores).
//                      Where the strip holds few of the rows of y its bands span (less than half), the
//                      lane that summed a row stores it through a 16-bit place inside the band instead.
//
// Per element: value + 16-bit column inside the slice (first pass), 16-bit LDS slot (second pass), and the
// product written once and read once; per bin a 32-bit shift, per row of y 16 bits.  No access to HBM is a
// gather.
#include "device_facts.hpp"
#include "templates.hpp"

namespace asx {
namespace tpl_shared_memory_product_bin {

static const uint64_t kUnit = 256;          // elements of one wavefront step (64 lanes x 4)
static const unsigned kBatch = 2;           // wavefront steps whose loads are in flight together
static const uint64_t kMaxRow = 4096;       // longest row the template takes: entries of a band's table of slot counts in LDS
static const uint64_t kNoRank = 0xffff;     // rank of a row of y that belongs to another strip
static const uint64_t kBandLdsBytes = 81920;  // LDS slots of a band: two workgroups of the second pass fit a CU
static const uint64_t kBinFlag = 0x8000;    // in a 16-bit slice column: first element of a bin
static const uint64_t kMaxTripBins = 4096;  // shifts of bins a trip of the first pass keeps in LDS (16 KB)

bool is_supported(const Matrix &m, uint64_t sub) {
  const DenseItem &it = m.items[sub];
  const CompressedBlock &cb = *it.cb;
  const uint64_t S = cb.col_slice, R = cb.row_group, vs = (uint64_t)dtype_size(m.val_dtype);
  // the slice of x and the shifts of a trip's bins share the LDS; a column needs 15 bits
  if (S == 0 || R == 0 || S > 32768 || R > 65536 || S % 4 || S * vs + kMaxTripBins * 4 > device_facts().lds_bytes) return false;
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
  std::vector<uint64_t> len(it.max_row - it.min_row + 1, 0);
  for (uint64_t r : row) len[r]++;
  const uint64_t longest = len.empty() ? 0 : *std::max_element(len.begin(), len.end());
  return longest <= kMaxRow;
}

std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  AS_CHECK(is_supported(m, sub), "format is not supported by SHARED_MEMORY_PRODUCT_BIN_TEMPLATE");
  const DenseItem &it = m.items[sub];
  const CompressedBlock &cb = *it.cb;
  const uint64_t S = cb.col_slice, H = cb.row_group, vs = (uint64_t)dtype_size(m.val_dtype);
  const std::vector<uint64_t> &row = cb.read_index[0]->index_arr.v, &col = cb.read_index[1]->index_arr.v;
  const ValVec &val = *cb.val;
  const uint64_t n = row.size(), sub_rows = it.max_row - it.min_row + 1, sub_cols = it.max_col - it.min_col + 1;
  const uint64_t nsl = (sub_cols + S - 1) / S;
  auto t = std::make_unique<Template>();
  init_template_common(*t, SHARED_MEMORY_PRODUCT_BIN_TEMPLATE, m, sub);
  t->is_atom_add = false;
  t->scalar["col_slice"] = S;
  t->scalar["row_group"] = H;
  t->scalar["sub_rows"] = sub_rows;
  t->scalar["slice_num"] = nsl;

  // row of y of every row of the sub-matrix (through the sort permutations when there are any), numbered from
  // the first row of y that the strip writes
  std::vector<uint64_t> y_row(sub_rows);
  for (uint64_t r = 0; r < sub_rows; r++) y_row[r] = r;
  t->global_sort_index = apply_global_sort(m, sub, y_row, sub_rows);
  if (!t->global_sort_index)
    for (uint64_t r = 0; r < sub_rows; r++) y_row[r] += it.min_row;
  const uint64_t y_base = *std::min_element(y_row.begin(), y_row.end());
  const uint64_t y_span = *std::max_element(y_row.begin(), y_row.end()) - y_base + 1;
  std::vector<uint32_t> row_of_y(y_span, 0xffffffffu);
  for (uint64_t r = 0; r < sub_rows; r++) {
    y_row[r] -= y_base;
    AS_CHECK(row_of_y[y_row[r]] == 0xffffffffu, "two rows of the strip share a row of y");
    row_of_y[y_row[r]] = (uint32_t)r;
  }
  std::vector<uint64_t> len(sub_rows, 0);
  for (uint64_t k = 0; k < n; k++) len[row[k]]++;
  const uint64_t longest = *std::max_element(len.begin(), len.end());

  // Bands: the rows of the strip in the order of y, cut where the next row of y lies H rows or more behind the
  // band's first (on the grid of multiples of H), where the band's elements would not fit its LDS slots any more,
  // or where its ranks would not fit 16 bits.  Inside a band the rows are ranked by falling length (rows of equal
  // length in the order of y).
  const uint64_t cap = std::max<uint64_t>(longest, std::min<uint64_t>(65535, kBandLdsBytes / vs) - 1);
  std::vector<uint64_t> band_first_row{0}, band_y_begin, band_y_end, trow;  // trow: rows of the strip in template order
  trow.reserve(sub_rows);
  {
    uint64_t y0 = 0, elems = 0;
    auto close_band = [&](uint64_t y_end) {
      std::stable_sort(trow.begin() + band_first_row.back(), trow.end(), [&](uint64_t a, uint64_t b) { return len[a] > len[b]; });
      band_y_begin.push_back(y0);
      band_y_end.push_back(y_end);
      band_first_row.push_back(trow.size());
      elems = 0;
    };
    for (uint64_t p = 0; p < y_span; p++) {
      const uint32_t r = row_of_y[p];
      if (r == 0xffffffffu) continue;
      const uint64_t rows_now = trow.size() - band_first_row.back();
      if (rows_now && p >= y0 + H) {
        close_band(y0 + H);
        y0 += (p - y0) / H * H;
      } else if (rows_now && (elems + len[r] > cap || rows_now + 1 > kNoRank)) {
        close_band(p);
        y0 = p;
      }
      trow.push_back(r);
      elems += len[r];
    }
    close_band(std::min(y0 + H, y_span));
  }
  const uint64_t nband = band_y_begin.size();
  std::vector<uint64_t> new_of_old(sub_rows), band_of_trow(sub_rows), rank_of_trow(sub_rows);
  uint64_t total_height = 0, max_height = 0, max_band_rows = 0;
  for (uint64_t b = 0; b < nband; b++) {
    for (uint64_t i = band_first_row[b]; i < band_first_row[b + 1]; i++) {
      new_of_old[trow[i]] = i;
      band_of_trow[i] = b;
      rank_of_trow[i] = i - band_first_row[b];
    }
    total_height += band_y_end[b] - band_y_begin[b];
    max_height = std::max(max_height, band_y_end[b] - band_y_begin[b]);
    max_band_rows = std::max(max_band_rows, band_first_row[b + 1] - band_first_row[b]);
  }
  // the strip holds at least half of the rows of y that its bands span: ranks by row of y, stores in the order of y
  const bool dense_y = total_height <= 2 * sub_rows;
  t->scalar["band_num"] = nband;
  t->scalar["dense_y"] = dense_y;
  t->scalar["y_base"] = y_base;
  t->scalar["max_band_height"] = max_height;
  t->scalar["max_band_rows"] = max_band_rows;

  // Slot counts of every band: first[j] = slots of the elements 0..j-1 of all its rows (rows longer than j' hold an
  // element j'), width + 1 entries, at least two.
  std::vector<uint64_t> band_first_jd(nband + 1, 0), band_jd, band_elems(nband, 0);
  for (uint64_t b = 0; b < nband; b++) {
    const uint64_t r0 = band_first_row[b], r1 = band_first_row[b + 1], width = std::max<uint64_t>(1, len[trow[r0]]);
    uint64_t longer = r1 - r0, first = 0;   // rows longer than j
    for (uint64_t j = 0; j <= width; j++) {
      band_jd.push_back(first);
      while (longer && len[trow[r0 + longer - 1]] <= j) longer--;
      first += longer;
    }
    band_elems[b] = band_jd.back();
    band_first_jd[b + 1] = band_jd.size();
  }
  t->scalar["max_width"] = std::max<uint64_t>(1, longest);

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

  // Second-pass stream: band by band, inside a band in the order of the first pass (slice by slice), every band
  // padded to whole units.  The padding is never written: it keeps the zeros of the upload and goes to a spare slot
  // behind the band's own.
  std::vector<uint64_t> band_first_unit(nband + 1, 0), fill(nband);
  uint64_t max_slots = 1;
  for (uint64_t b = 0; b < nband; b++) {
    band_first_unit[b + 1] = band_first_unit[b] + (band_elems[b] + kUnit - 1) / kUnit;
    fill[b] = band_first_unit[b] * kUnit;
    max_slots = std::max(max_slots, band_elems[b] + 1);
  }
  const uint64_t product_len = band_first_unit[nband] * kUnit;
  AS_CHECK(product_len < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
  AS_CHECK(max_slots <= 65536 && max_slots * vs + (t->sc("max_width") + 1) * 4 <= device_facts().lds_bytes,
           "a band does not fit its LDS slots");
  std::vector<uint64_t> slot(product_len);
  for (uint64_t b = 0; b < nband; b++)
    std::fill(slot.begin() + band_first_unit[b] * kUnit, slot.begin() + band_first_unit[b + 1] * kUnit, band_elems[b]);

  // First-pass stream slice by slice, every slice padded to whole units.  The elements of one slice and one band
  // (a bin) are consecutive in the stream and go to consecutive places of the band's products, so a place is not
  // stored per element: the first element of a bin carries a flag (the top bit of its 16-bit column), a unit knows
  // how many bins start before it, and a bin knows how far its products lie from its elements (`bin_shift`, modulo
  // 2^32).  The padding of a slice is a bin of its own whose products land in a spare stretch behind the last band.
  std::vector<uint64_t> lcol, slice_first_unit(nsl + 1, 0), seen(sub_rows, 0), bin_shift, unit_first_bin;
  lcol.reserve(n + nsl * kUnit);
  t->val_arr.reserve(n + nsl * kUnit);
  uint64_t cur_slice = 0, cur_band = ~0ull;
  auto open_bin = [&](uint64_t place) {
    bin_shift.push_back((place - lcol.size()) & 0xffffffffull);
    return kBinFlag;
  };
  auto push = [&](uint64_t column, double value) {
    if (lcol.size() % kUnit == 0) unit_first_bin.push_back(bin_shift.size() - (column & kBinFlag ? 1 : 0));
    lcol.push_back(column);
    t->val_arr.push_back(value);
  };
  auto close_slices_up_to = [&](uint64_t s) {  // pad the open slice, give empty slices an empty unit range
    while (cur_slice < s) {
      for (bool first = true; lcol.size() % kUnit; first = false) push(first ? open_bin(product_len) : 0, 0.0);
      slice_first_unit[++cur_slice] = lcol.size() / kUnit;
      cur_band = ~0ull;
    }
  };
  for (uint64_t i = 0; i < n; i++) {
    const uint64_t k = order[i], s = col[k] / S, tr = new_of_old[row[k]], b = band_of_trow[tr];
    close_slices_up_to(s);
    uint64_t flag = 0;
    if (b != cur_band) {
      flag = open_bin(fill[b]);
      cur_band = b;
    }
    push((col[k] - s * S) | flag, val[k]);
    slot[fill[b]++] = band_jd[band_first_jd[b] + seen[tr]++] + rank_of_trow[tr];
  }
  close_slices_up_to(nsl);
  const uint64_t padded = lcol.size();
  AS_CHECK(padded < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
  unit_first_bin.push_back(bin_shift.size());
  t->scalar["max_slots"] = max_slots;
  t->scalar["max_band_units"] = (max_slots - 1 + kUnit - 1) / kUnit;
  t->col_index_arr.assign(std::move(lcol), UNSIGNED_SHORT);
  t->scratch_bytes = (product_len + kUnit) * vs;
  t->scalar["product_len"] = product_len;

  // first pass: trips of about equal cost (units of elements + one slice copy each), cut inside slices; a trip
  // keeps the shifts of its bins in LDS, at most kMaxTripBins of them
  const uint64_t lds = device_facts().lds_bytes, cus = device_facts().cu_num;
  const uint64_t unit_bytes = kUnit * (2 * vs + 2), slice_units = (S * vs + unit_bytes - 1) / unit_bytes;
  const uint64_t total_units = padded / kUnit;
  uint64_t want = cus * std::max<uint64_t>(1, lds / (S * vs));
  want = std::max<uint64_t>(1, std::min<uint64_t>(want, (total_units + 63) / 64));
  uint64_t nonempty = 0;
  for (uint64_t s = 0; s < nsl; s++) nonempty += slice_first_unit[s + 1] > slice_first_unit[s];
  const uint64_t per_trip = (total_units + (nonempty + want) * slice_units) / want + 1;
  std::vector<uint64_t> group_slice, group_first_unit;
  uint64_t max_trip_bins = 1;
  // bins a trip of the units [u, e) reads: from the one its first element lies in to the last one that starts in it
  auto trip_bins = [&](uint64_t u, uint64_t e) { return unit_first_bin[e] - (unit_first_bin[u] ? unit_first_bin[u] - 1 : 0); };
  for (uint64_t s = 0; s < nsl; s++) {
    uint64_t u0 = slice_first_unit[s], u1 = slice_first_unit[s + 1];
    if (u1 == u0) continue;
    uint64_t room = per_trip > slice_units ? per_trip - slice_units : 1;
    uint64_t parts = std::max<uint64_t>(1, (u1 - u0 + room / 2) / room), per = (u1 - u0 + parts - 1) / parts;
    for (uint64_t u = u0; u < u1;) {
      uint64_t e = std::min(u1, u + per);
      while (e > u + 1 && trip_bins(u, e) > kMaxTripBins) e = u + (e - u + 1) / 2;
      group_slice.push_back(s);
      group_first_unit.push_back(u);
      max_trip_bins = std::max(max_trip_bins, trip_bins(u, e));
      u = e;
    }
  }
  // a trip ends where the next one starts; the last one at the end of its slice, which is where the
  // next non-empty slice starts
  group_first_unit.push_back(total_units);
  t->scalar["group_num"] = group_slice.size();
  t->scalar["max_trip_bins"] = max_trip_bins;
  AS_CHECK(max_trip_bins <= kMaxTripBins, "a unit of the first pass holds more bins than a trip keeps in LDS");

  auto add = [&](const char *name, std::vector<uint64_t> v, DType at_least) {
    TArr a;
    a.name = name;
    uint64_t mx = v.empty() ? 0 : *std::max_element(v.begin(), v.end());
    a.a.assign(std::move(v), IArr::at_least(at_least, mx));
    t->arrays.push_back(std::move(a));
  };
  add("group_slice", std::move(group_slice), UNSIGNED_CHAR);
  add("group_first_unit", std::move(group_first_unit), UNSIGNED_CHAR);
  add("unit_first_bin", std::move(unit_first_bin), UNSIGNED_INT);   // read with scalar loads
  add("bin_shift", std::move(bin_shift), UNSIGNED_INT);
  // read with scalar loads, which need 32-bit entries
  add("band_first_unit", std::move(band_first_unit), UNSIGNED_INT);
  add("band_first_count", std::move(band_first_jd), UNSIGNED_INT);
  add("band_y_begin", std::move(band_y_begin), UNSIGNED_INT);
  if (dense_y) {
    add("band_y_end", std::move(band_y_end), UNSIGNED_INT);
  } else {
    add("band_first_row", std::move(band_first_row), UNSIGNED_INT);
  }
  add("band_slot_count", std::move(band_jd), UNSIGNED_SHORT);
  add("slot_in_band", std::move(slot), UNSIGNED_SHORT);
  if (dense_y) {
    std::vector<uint64_t> rank_of_y(y_span, kNoRank);
    for (uint64_t i = 0; i < sub_rows; i++) rank_of_y[y_row[trow[i]]] = rank_of_trow[i];
    add("rank_of_y_row", std::move(rank_of_y), UNSIGNED_SHORT);
  } else {
    std::vector<uint64_t> y_of_rank(sub_rows);
    const IArr &y_begin_of_band = t->find("band_y_begin")->a;
    for (uint64_t i = 0; i < sub_rows; i++) y_of_rank[i] = y_row[trow[i]] - y_begin_of_band[band_of_trow[i]];
    add("y_row_of_rank", std::move(y_of_rank), UNSIGNED_SHORT);
  }
  tpl_shared_memory_product_bin::set_default_launch(*t);
  return t;
}

void try_all_compress(Template &t) {
  for (const char *name : {"group_first_unit", "unit_first_bin", "band_first_unit", "band_first_count", "band_y_begin", "band_y_end", "band_first_row"}) {
    TArr *a = t.find(name);
    if (a && !a->c.active()) init_linear_compressor(a->a, a->c, true);
  }
  TArr &s = *t.find("group_slice");
  if (!s.c.active() && !init_linear_compressor(s.a, s.c, true)) init_cycle_increase_compressor(s.a, s.c, true);
}

void set_default_launch(Template &t) {
  const uint64_t vs = (uint64_t)dtype_size(t.val_dtype);
  if (t.thread_num_in_block == 0) t.thread_num_in_block = 1024;
  t.tblock_num = std::max<uint64_t>(1, std::min<uint64_t>(t.sc("group_num"), (1ull << 31) - 1));
  t.dynamic_lds_bytes = t.sc("col_slice") * vs + t.sc("max_trip_bins") * 4;
  t.finish_tblock_num = std::max<uint64_t>(1, std::min<uint64_t>(t.sc("band_num"), (1ull << 31) - 1));
  // a lane for every fourth row of the tallest band, between 256 and 1024 (C3, bands of 4096 rows of y: second
  // pass 17.0 / 12.6 / 10.8 us with 256 / 512 / 1024 lanes)
  t.finish_thread_num = std::min<uint64_t>(1024, std::max<uint64_t>(256, (t.sc("max_band_rows") / 4 + 63) / 64 * 64));
  t.finish_lds_bytes = t.sc("max_slots") * vs;
}

std::string kernel_source(const Template &t) {
  const std::string vt = value_type_name(t);
  AS_CHECK(t.col_index_arr.dt == UNSIGNED_SHORT && t.arr("slot_in_band").a.dt == UNSIGNED_SHORT &&
               t.arr("bin_shift").a.dt == UNSIGNED_INT, "slice columns and LDS slots must be 16 bits wide, shifts 32");
  AS_CHECK(t.thread_num_in_block % 64 == 0 && t.thread_num_in_block >= 64 && t.thread_num_in_block <= 1024,
           "thread_num_in_block must be a multiple of 64 up to 1024");
  const uint64_t S = t.sc("col_slice"), G = t.sc("group_num"), nband = t.sc("band_num");
  const bool dense_y = t.sc("dense_y") != 0;
  const std::string id = std::to_string(t.sub), B = std::to_string(t.thread_num_in_block) + "u";
  const std::string Ss = std::to_string(S) + "u", Ks = std::to_string(kBatch);
  const std::string FB = std::to_string(t.finish_thread_num);
  const uint64_t x_len = t.matrix_cols - t.kernal_first_col_index;
  const bool wide_copy = t.kernal_first_col_index % 4 == 0;
  std::string s;
  // ---- first pass: products -------------------------------------------------------------------
  // Fused launch: the workgroups first run the trips of the strip in front of this one (its arrays behind this
  // kernel's own, `fused_on` = 0 when this strip is launched alone), then their own; the carried finish is then the
  // second kernel's.  Otherwise the first workgroups of this kernel carry the finish (carried_finish_prologue).
  const Template *fused = t.fused_trips;
  AS_CHECK(!fused || (fused == t.carried && fused->thread_num_in_block == t.thread_num_in_block),
           "a fused launch needs the same workgroup size in both strips");
  s += "extern \"C\" __global__ void __launch_bounds__(" + std::to_string(t.thread_num_in_block) + ") spmv_" + id + "(" +
       kernel_signature(t) + (fused ? ", " + kernel_signature(*fused, "fused_") + ", unsigned int fused_on" : carried_finish_signature(t)) + ")\n{\n";
  if (fused) {
    // The launch has as many workgroups as the longer of the two lists of trips.  Each list is dealt out among its
    // own first workgroups only (workgroup i runs on XCD i % 8, and the XCD-contiguous numbering of the trips
    // assumes that the workgroups that share them are numbered 0, 1, 2, ...): numbered over the whole launch, the
    // trips of the shorter list would all land on the first XCDs.
    const std::string G0 = std::to_string(fused->tblock_num) + "u";
    s += "  if (fused_on && blockIdx.x < " + G0 + ")\n  {\n    " + kernel_trips_function_name(*fused) + "(" + kernel_arguments(*fused, "fused_") + ", blockIdx.x, " + G0 + ");\n";
    s += "    as_barrier();\n  }\n";   // the LDS is this kernel's from here on
    s += "  const unsigned int as_block = blockIdx.x, as_grid = min(gridDim.x, " + std::to_string(t.tblock_num) + "u);\n";
    s += "  if (as_block >= as_grid) return;\n";
  } else {
    s += carried_finish_prologue(t, t.thread_num_in_block);
  }
  const std::string Cs = std::to_string(16 / dtype_size(t.val_dtype));
  s += "  typedef " + vt + " val16_t __attribute__((ext_vector_type(" + Cs + ")));\n";  // 16 bytes of values
  s += "  extern __shared__ __attribute__((aligned(16))) unsigned char as_dynamic_lds[];\n";
  s += "  " + vt + " *x_slice = (" + vt + " *)as_dynamic_lds;\n";
  s += "  unsigned int *shift_of_bin = (unsigned int *)(as_dynamic_lds + " + std::to_string(S * dtype_size(t.val_dtype)) + "u);\n";
  s += "  " + vt + " *product = (" + vt + " *)scratch_arr;\n";
  s += "  const unsigned int lane = threadIdx.x & 63u, wave_in_block = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);\n";
  s += "  const unsigned int stride = (" + B + " >> 6) * 256u;\n";
  s += "  const " + vt + " *x_sub = device_x_arr + " + std::to_string(t.kernal_first_col_index) + "u;\n";
  s += "  for (unsigned int grp = as_xcd_block_index(as_block, as_grid); grp < " + std::to_string(G) + "u; grp += as_grid)\n  {\n";
  s += "    unsigned int next_grp = grp + 1u, slice, unit_begin, unit_end, bins_before, bins_end;\n";
  s += "    " + code_of_meta_read(t, "group_slice", "slice", "grp");
  s += "    " + code_of_meta_read(t, "group_first_unit", "unit_begin", "grp");
  s += "    " + code_of_meta_read(t, "group_first_unit", "unit_end", "next_grp");
  s += "    " + code_of_meta_read(t, "unit_first_bin", "bins_before", "unit_begin");
  s += "    " + code_of_meta_read(t, "unit_first_bin", "bins_end", "unit_end");
  // the trip's bins: from the one its first element lies in (started before it, unless the element opens one)
  s += "    const unsigned int bin0 = bins_before ? bins_before - 1u : 0u;\n";
  s += "    const unsigned int col0 = slice * " + Ss + ";\n";
  s += "    const unsigned int slice_len = min(" + Ss + ", " + std::to_string(x_len) + "u - col0);\n";
  s += "    as_barrier();\n";  // readers of the previous slice are done
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
  s += "    for (unsigned int i = threadIdx.x; i < bins_end - bin0; i += " + B + ") shift_of_bin[i] = bin_shift[bin0 + i];\n";
  s += "    as_barrier();\n";
  // Consecutive lanes take consecutive elements: the products of a bin then go to consecutive places with one
  // store instruction (whole lines), instead of every fourth place with each of four.  A lane finds the bin of its
  // element by counting the flags of the elements before it: those of the unit's earlier loads (a scalar), those
  // of the lower lanes of its own load (ballot + mbcnt).
  s += "    const unsigned int nz_end = unit_end * 256u;\n";
  s += "    for (unsigned int nz0 = unit_begin * 256u + wave_in_block * 256u; nz0 < nz_end; nz0 += stride * " + Ks + "u)\n    {\n";
  s += "      " + vt + " a[" + Ks + "][4];\n      unsigned short c[" + Ks + "][4];\n      unsigned int started[" + Ks + "];\n";
  s += "      #pragma unroll\n      for (int k = 0; k < " + Ks + "; k++)\n      {\n";
  s += "        if (nz0 + k * stride < nz_end)\n        {\n";
  s += "          const unsigned int unit = (nz0 + k * stride) >> 8;\n";
  s += "          " + code_of_meta_read(t, "unit_first_bin", "started[k]", "unit");
  s += "          #pragma unroll\n          for (int j = 0; j < 4; j++)\n          {\n";
  s += "            const unsigned int nz = nz0 + k * stride + j * 64u + lane;\n";
  s += "            a[k][j] = as_ldnt(val_arr + nz);\n";
  s += "            c[k][j] = as_ldnt(col_index_arr + nz);\n";
  s += "          }\n        }\n      }\n";
  s += "      #pragma unroll\n      for (int k = 0; k < " + Ks + "; k++)\n      {\n";
  s += "        if (nz0 + k * stride < nz_end)\n        {\n";
  s += "          unsigned int before = __builtin_amdgcn_readfirstlane(started[k]) - bin0 - 1u;\n";
  s += "          #pragma unroll\n          for (int j = 0; j < 4; j++)\n          {\n";
  s += "            const unsigned int flag = (unsigned int)c[k][j] >> 15;\n";
  s += "            const unsigned long long opened = __builtin_amdgcn_ballot_w64(flag != 0u);\n";
  s += "            const unsigned int upto = __builtin_amdgcn_mbcnt_hi((unsigned int)(opened >> 32), __builtin_amdgcn_mbcnt_lo((unsigned int)opened, 0u)) + flag;\n";
  s += "            const unsigned int shift = shift_of_bin[before + upto];\n";
  s += "            before += (unsigned int)__builtin_popcountll(opened);\n";
  s += "            product[nz0 + k * stride + j * 64u + lane + shift] = a[k][j] * x_slice[(unsigned int)c[k][j] & 32767u];\n";
  s += "          }\n";
  s += "        }\n      }\n    }\n  }\n}\n";
  // ---- second pass: row sums ------------------------------------------------------------------
  const uint64_t FBn = t.finish_thread_num;
  // ranks (rows of y) of a lane that are requested before the products
  const unsigned ahead = (unsigned)std::min<uint64_t>(8, std::max<uint64_t>(1, (t.sc("max_band_height") + FBn - 1) / FBn));
  const std::string As = std::to_string(ahead), Ybase = std::to_string(t.sc("y_base")) + "u";
  // wavefront steps of the second pass whose loads are in flight together: as many as a wavefront has in the
  // largest band, up to four -- a band is then streamed in one round trip to memory
  const unsigned batch2 = (unsigned)std::min<uint64_t>(4, std::max<uint64_t>(1, (t.sc("max_band_units") + FBn / 64 - 1) / (FBn / 64)));
  const std::string K2 = std::to_string(batch2);
  // The band's table of slot counts (first[j], j = 0 .. width) lives in a register where no row has more than 63
  // elements: lane j of every wavefront holds first[j], read with v_readlane -- no LDS round trip between two
  // elements of a row.  Wider rows: a table in LDS.
  const bool table_in_register = t.sc("max_width") <= 63;
  s += "extern \"C\" __global__ void __launch_bounds__(" + FB + ") spmv_" + id + "_finish(" + kernel_signature(t) +
       (fused ? carried_finish_signature(t) : std::string()) + ")\n{\n";
  if (fused) s += carried_finish_prologue(t, FBn);
  else s += "  const unsigned int as_block = blockIdx.x, as_grid = gridDim.x;\n";
  s += "  extern __shared__ __attribute__((aligned(16))) unsigned char as_dynamic_lds[];\n";
  if (!table_in_register) s += "  __shared__ unsigned int first_slot[" + std::to_string(t.sc("max_width") + 1) + "];\n";
  s += "  " + vt + " *slots = (" + vt + " *)as_dynamic_lds;\n";
  s += "  const " + vt + " *product = (const " + vt + " *)scratch_arr;\n";
  s += "  const unsigned int lane = threadIdx.x & 63u, wave_in_block = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);\n";
  s += "  const unsigned int stride = (" + FB + "u >> 6) * 256u;\n";
  // neighbouring bands write neighbouring rows of y: they run on the same XCD, behind the same L2
  s += "  for (unsigned int grp = as_xcd_block_index(as_block, as_grid); grp < " + std::to_string(nband) + "u; grp += as_grid)\n  {\n";
  s += "    unsigned int next_grp = grp + 1u, unit_begin, unit_end, count_begin, count_end, y_begin;\n";
  s += "    " + code_of_meta_read(t, "band_first_unit", "unit_begin", "grp");
  s += "    " + code_of_meta_read(t, "band_first_unit", "unit_end", "next_grp");
  s += "    " + code_of_meta_read(t, "band_first_count", "count_begin", "grp");
  s += "    " + code_of_meta_read(t, "band_first_count", "count_end", "next_grp");
  s += "    " + code_of_meta_read(t, "band_y_begin", "y_begin", "grp");
  s += "    const unsigned int width = count_end - count_begin - 1u;\n";
  if (table_in_register) s += "    const unsigned int first_of_lane = band_slot_count[count_begin + min(lane, width)];\n";
  if (dense_y) {
    s += "    unsigned int y_end;\n";
    s += "    " + code_of_meta_read(t, "band_y_end", "y_end", "grp");
    s += "    const unsigned int height = y_end - y_begin;\n";
    // the ranks of the lane's first rows of y are requested now and used after the sums
    s += "    unsigned short rank[" + As + "];\n";
    s += "    #pragma unroll\n    for (int k = 0; k < " + As + "; k++) rank[k] = rank_of_y_row[y_begin + min(threadIdx.x + k * " + FB + "u, height - 1u)];\n";
  } else {
    s += "    unsigned int row_begin, row_end;\n";
    s += "    " + code_of_meta_read(t, "band_first_row", "row_begin", "grp");
    s += "    " + code_of_meta_read(t, "band_first_row", "row_end", "next_grp");
  }
  s += "    as_barrier();\n";  // the previous band's sums have been read
  if (!table_in_register)
    s += "    for (unsigned int i = threadIdx.x; i <= width; i += " + FB + "u) first_slot[i] = band_slot_count[count_begin + i];\n";
  s += "    const unsigned int nz_end = unit_end * 256u;\n";
  s += "    for (unsigned int nz0 = unit_begin * 256u + wave_in_block * 256u; nz0 < nz_end; nz0 += stride * " + K2 + "u)\n    {\n";
  // consecutive lanes take consecutive products: every load of the 64 lanes reads one contiguous stretch
  s += "      " + vt + " p[" + K2 + "][4];\n      unsigned short q[" + K2 + "][4];\n";
  s += "      #pragma unroll\n      for (int k = 0; k < " + K2 + "; k++)\n      {\n";
  s += "        if (nz0 + k * stride < nz_end)\n        {\n";
  s += "          #pragma unroll\n          for (int j = 0; j < 4; j++)\n          {\n";
  s += "            const unsigned int nz = nz0 + k * stride + j * 64u + lane;\n";
  s += "            p[k][j] = product[nz];\n";
  s += "            q[k][j] = as_ldnt(slot_in_band + nz);\n";
  s += "          }\n        }\n      }\n";
  s += "      #pragma unroll\n      for (int k = 0; k < " + K2 + "; k++)\n      {\n";
  s += "        if (nz0 + k * stride >= nz_end) continue;\n";
  s += "        #pragma unroll\n        for (int j = 0; j < 4; j++) slots[(unsigned int)q[k][j]] = p[k][j];\n";
  s += "      }\n    }\n";
  s += "    as_barrier();\n";
  // Row sums: lane r0 + lane of a wavefront takes the row of that rank; rows are ranked by falling length, so the
  // wavefront is done where its first row is (a test on scalars).  Rows without elements have the last ranks.
  // Four elements of a row are requested from LDS before the first is added.
  const std::string first_of = table_in_register ? "(unsigned int)__builtin_amdgcn_readlane((int)first_of_lane, (int)min(" : "__builtin_amdgcn_readfirstlane(first_slot[min(";
  const std::string first_end = table_in_register ? ", width))" : ", width)])";
  s += "    const unsigned int live = " + first_of + "1u" + first_end + ";\n";
  const std::string bound = dense_y ? "live" : "row_end - row_begin";
  s += "    for (unsigned int r0 = wave_in_block * 64u; r0 < " + bound + "; r0 += " + FB + "u)\n    {\n";
  s += "      const unsigned int r = r0 + lane;\n";
  s += "      " + vt + " sum = 0;\n";
  s += "      unsigned int f0 = 0u;\n";
  s += "      for (unsigned int j = 0; j < width; j += 4u)\n      {\n";
  s += "        const unsigned int f1 = " + first_of + "j + 1u" + first_end + ", f2 = " + first_of + "j + 2u" + first_end +
       ", f3 = " + first_of + "j + 3u" + first_end + ", f4 = " + first_of + "j + 4u" + first_end + ";\n";
  s += "        if (f1 - f0 <= r0) break;\n";
  s += "        const " + vt + " a0 = r < f1 - f0 ? slots[f0 + r] : (" + vt + ")0, a1 = r < f2 - f1 ? slots[f1 + r] : (" + vt + ")0;\n";
  s += "        const " + vt + " a2 = r < f3 - f2 ? slots[f2 + r] : (" + vt + ")0, a3 = r < f4 - f3 ? slots[f3 + r] : (" + vt + ")0;\n";
  s += "        sum += a0;\n        sum += a1;\n        sum += a2;\n        sum += a3;\n";
  s += "        f0 = f4;\n";
  s += "      }\n";
  if (dense_y) {
    // slot r is the row's own first element: nobody else reads it
    s += "      if (r < live) slots[r] = sum;\n";
    s += "    }\n";
    s += "    as_barrier();\n";
    s += "    #pragma unroll\n    for (int k = 0; k < " + As + "; k++)\n    {\n";
    s += "      const unsigned int i = threadIdx.x + k * " + FB + "u;\n";
    s += "      if (i < height && rank[k] != " + std::to_string(kNoRank) + "u)\n";
    s += "        as_stnt(device_y_arr + " + Ybase + " + y_begin + i, rank[k] < live ? slots[(unsigned int)rank[k]] : (" + vt + ")0);\n";
    s += "    }\n";
    s += "    for (unsigned int i = threadIdx.x + " + As + "u * " + FB + "u; i < height; i += " + FB + "u)\n    {\n";
    s += "      const unsigned int rk = rank_of_y_row[y_begin + i];\n";
    s += "      if (rk != " + std::to_string(kNoRank) + "u) as_stnt(device_y_arr + " + Ybase + " + y_begin + i, rk < live ? slots[rk] : (" + vt + ")0);\n";
    s += "    }\n";
  } else {
    s += "      if (r < row_end - row_begin) as_stnt(device_y_arr + " + Ybase + " + y_begin + (unsigned int)y_row_of_rank[row_begin + r], sum);\n";
    s += "    }\n";
  }
  s += "  }\n}\n";
  return s;
}

}  // namespace tpl_shared_memory_product_bin
}  // namespace asx
