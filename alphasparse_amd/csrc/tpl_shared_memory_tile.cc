// SHARED_MEMORY_TILE_TEMPLATE (no upstream counterpart): rows whose columns are spread over a
// vector much larger than the L2 cache.  The BLBs are 2-D tiles -- rows of one row group, columns of
// one column slice (COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE_PARAM_STRATEGY) -- stored
// tile by tile.  A workgroup keeps the slice of x (col_slice values) and the partial sums of the row
// group (row_group values) in LDS, 160 KB together at the default sizes, so that every x read and
// every row sum of an element is an LDS access; HBM sees the element stream (one 128-bit load of
// values and one of packed indices per lane and trip), one copy of the slice per workgroup trip and
// one atomic per row and trip when the row group is written back.
//
// The element stream is cut into `group_num` workgroup trips of about equal cost (elements plus the
// slice copies and write-backs the trip causes); consecutive BLBs of one tile inside a trip form a
// run, padded to a multiple of 512 elements with zeros on the run's last row.  Inside a run every
// row is one piece of consecutive elements, and the pieces are numbered 0, 1, 2, ...: the LDS cell of
// a piece is its number, and a table gives the place of every piece in y (or in the dense scratch
// vector) for the write-back at the end of the run.
//
// An element is val + a 16-bit column inside the slice; a lane takes 8 consecutive elements and one
// 32-bit word for them all: the piece of its first element (15 bits), for each of the other seven
// whether it starts a new piece, and for each of the eight whether a sum emitted there may be stored.
// That is 6.5 bytes per fp32 element and 10.5 per fp64 element; the kernel's time follows its bytes.
// The lane adds up the pieces that end inside its eight elements, and the wavefront merges the
// pieces that continue across lanes with a segmented scan by DPP (piece numbers are sorted along
// the lanes), so a piece costs one LDS access per wavefront step however long it is.
//
// Column-run form (init(..., column_runs = true)): where the columns of a lane's eight elements come in a few
// runs of consecutive columns (dense blocks of a FEM matrix, dense rows), the lane stores the first column of
// up to four runs (4 x 16 bits) and one byte whose bit j says that element j starts the next run; the other
// columns are the previous one plus 1.  That is 9 bytes of columns per lane instead of 16 (fp64 element: 9.625
// bytes instead of 10.5).  A lane that would need a fifth run is closed with zero-valued elements and the run
// opens the next lane; a run start beyond the fourth decodes as column 0, which is where padding points.
//
// Row ownership (init_variant(..., own_rows = true)): where the matrix has many row groups that each meet few
// columns (banded matrices), a trip is a whole number of row groups and the elements are taken row group by row
// group, inside a group window by window of x (a window starts at the group's first column not yet covered and is
// col_slice columns wide), inside a window row by row.  The LDS cell of a row is its place in the group and lives
// across the group's runs; at the end of a group the workgroup stores the group's rows to y: no atomics into y,
// no table of places, no scratch vector, no finish kernel, no clear of y.
//
// Row blocks (init_variant(..., row_block = b), under row ownership): where b consecutive rows hold the same
// columns (the dense b x b blocks of a FEM matrix), a block of rows is one piece: columns, lane word and reads of
// x are those of its first row, an element is b values, and a lane adds into b sums.
#include "device_facts.hpp"
#include "templates.hpp"

namespace asx {
namespace tpl_shared_memory_tile {

static const unsigned kLaneRuns = 4;        // column runs a lane of the column-run form can hold

static const uint64_t kLaneElems = 8;       // consecutive elements of one lane in a wavefront step
static const uint64_t kRunUnit = 64 * kLaneElems;  // elements of one wavefront step
static const unsigned kNewPieceBit = 14;    // lane word: bit 14 + j = element j (1..7) starts a new piece
static const unsigned kStoreBit = 14 + kLaneElems;  // bit 22 + j = a sum emitted at element j (0..7) is the piece's only one
static const unsigned kBetweenRunsBatch = 8; // requests a lane keeps in flight in the write-back and in the slice copy
static const unsigned kBatch = 1;           // wavefront steps whose loads are in flight together (a step is 8
                                            // elements per lane, 4-6 loads: deeper batches measured slower)

bool is_supported(const Matrix &m, uint64_t sub) {
  const DenseItem &it = m.items[sub];
  const CompressedBlock &cb = *it.cb;
  const uint64_t S = cb.col_slice, R = cb.row_group, vs = (uint64_t)dtype_size(m.val_dtype);
  if (S == 0 || R == 0 || S > 65536 || R > 32768 || S % 4 || (S + R) * vs > device_facts().lds_bytes) return false;
  if (it.max_row != cb.read_index[0]->max_row) return false;  // not after COMPRESSED_ROW_PADDING
  const Index &bl = *cb.read_index[2];
  const std::vector<uint64_t> &row = cb.read_index[0]->index_arr.v, &col = cb.read_index[1]->index_arr.v;
  if (bl.block_num == 0 || bl.coo_begin[bl.block_num] != row.size()) return false;
  for (uint64_t b = 0; b < bl.block_num; b++) {
    uint64_t k0 = bl.coo_begin[b], k1 = bl.coo_begin[b + 1];
    if (k1 <= k0) return false;
    for (uint64_t k = k0 + 1; k < k1; k++)
      if (col[k] / S != col[k0] / S || row[k] / R != row[k0] / R || row[k] < row[k - 1]) return false;
  }
  return true;
}

static std::unique_ptr<Template> build(const Matrix &m, uint64_t sub, bool column_runs, bool own_rows, uint64_t row_block = 1);

// Elements the stream of the column-run form would hold, lane-closing padding included (the padding of runs to whole
// wavefront steps left out): one pass over the columns, nothing built.  A lane takes eight elements and at most
// kLaneRuns runs of consecutive columns; tiles start on a new lane.
uint64_t column_run_stream_estimate(const Matrix &m, uint64_t sub) {
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &bl = *cb.read_index[2];
  const uint64_t S = cb.col_slice, R = cb.row_group;
  const std::vector<uint64_t> &row = cb.read_index[0]->index_arr.v, &col = cb.read_index[1]->index_arr.v;
  uint64_t total = 0, fill = 0, runs = 0, prev = 0;
  for (uint64_t b = 0; b < bl.block_num; b++) {
    const uint64_t k0 = bl.coo_begin[b], k1 = bl.coo_begin[b + 1];
    if (b > 0 && (col[k0] / S != col[bl.coo_begin[b - 1]] / S || row[k0] / R != row[bl.coo_begin[b - 1]] / R) && fill) {
      total += kLaneElems - fill;
      fill = 0;
    }
    for (uint64_t k = k0; k < k1; k++) {
      if (fill == 0) runs = 0;
      if (fill == 0 || col[k] != prev + 1) {
        if (runs >= kLaneRuns) {
          total += kLaneElems - fill;
          fill = 0;
          runs = 0;
        }
        runs++;
      }
      prev = col[k];
      total++;
      fill = (fill + 1) % kLaneElems;
    }
  }
  return total + (fill ? kLaneElems - fill : 0);
}
std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) { return build(m, sub, false, false); }
std::unique_ptr<Template> init_with_column_runs(const Matrix &m, uint64_t sub) { return build(m, sub, true, false); }
// nullptr when row ownership does not fit the sub-matrix (see build)
std::unique_ptr<Template> init_variant(const Matrix &m, uint64_t sub, bool column_runs, bool own_rows, uint64_t row_block) {
  return build(m, sub, column_runs, own_rows, row_block);
}

// The height of the blocks of rows the sub-matrix seems to be made of, from the rows of its first tile (up to 16
// blocks): 4, 3 or 2 where that many consecutive rows (the first a multiple of the height, the height a divisor of
// the row group's) hold the same columns block after block, else 1.  A guess that saves building a form that cannot
// apply; the build itself checks every block.
uint64_t row_block_guess(const Matrix &m, uint64_t sub) {
  const CompressedBlock &cb = *m.items[sub].cb;
  const Index &bl = *cb.read_index[2];
  const uint64_t S = cb.col_slice, R = cb.row_group;
  const std::vector<uint64_t> &row = cb.read_index[0]->index_arr.v, &col = cb.read_index[1]->index_arr.v;
  uint64_t blbs = 1;
  while (blbs < bl.block_num && col[bl.coo_begin[blbs]] / S == col[bl.coo_begin[0]] / S &&
         row[bl.coo_begin[blbs]] / R == row[bl.coo_begin[0]] / R)
    blbs++;
  const uint64_t k0 = bl.coo_begin[0], k1 = bl.coo_begin[blbs];
  std::vector<uint64_t> start;
  for (uint64_t k = k0; k < k1 && start.size() <= 64; k++)
    if (k == k0 || row[k] != row[k - 1]) start.push_back(k);
  if (start.size() <= 64) start.push_back(k1);
  const uint64_t rows = start.size() - 1;
  for (uint64_t h : {4, 3, 2}) {
    if (R % h != 0 || rows < h) continue;
    bool same = true;
    for (uint64_t blk = 0; same && blk < std::min<uint64_t>(rows / h, 16); blk++) {
      const uint64_t f = blk * h, len = start[f + 1] - start[f];
      same = row[start[f]] % h == 0;
      for (uint64_t q = 1; same && q < h; q++) {
        same = row[start[f + q]] == row[start[f]] + q && start[f + q + 1] - start[f + q] == len;
        for (uint64_t e = 0; same && e < len; e++) same = col[start[f + q] + e] == col[start[f] + e];
      }
    }
    if (same) return h;
  }
  return 1;
}

static std::unique_ptr<Template> build(const Matrix &m, uint64_t sub, bool column_runs, bool own_rows, uint64_t row_block) {
  AS_CHECK(is_supported(m, sub), "format is not supported by SHARED_MEMORY_TILE_TEMPLATE");
  AS_CHECK(row_block >= 1 && row_block <= 4, "row blocks of 1 to 4 rows");
  // Row blocks (row_block = b > 1, under row ownership): b consecutive rows (b divides the row's number and the
  // row group's height) that hold the same columns are one piece of the stream -- the columns, the lane word and
  // the x reads are those of the first row, and an element is b values, one per row.  Dense b x b blocks of a FEM
  // matrix: 8 bytes of columns + 1 of run starts + 4 of lane word per 8 b elements.  nullptr where a block of rows
  // does not hold the same columns in a window.
  const DenseItem &it = m.items[sub];
  const CompressedBlock &cb = *it.cb;
  const Index &bl = *cb.read_index[2];
  const uint64_t S = cb.col_slice, R = cb.row_group, B = bl.block_num, vs = (uint64_t)dtype_size(m.val_dtype);
  if (row_block > 1 && (!own_rows || R % row_block != 0)) return nullptr;
  const std::vector<uint64_t> &row = cb.read_index[0]->index_arr.v, &col = cb.read_index[1]->index_arr.v;
  const ValVec &val = *cb.val;
  const uint64_t n = row.size(), sub_rows = it.max_row - it.min_row + 1;
  auto t = std::make_unique<Template>();
  init_template_common(*t, SHARED_MEMORY_TILE_TEMPLATE, m, sub);
  t->is_atom_add = true;
  t->scalar["col_slice"] = S;
  t->scalar["row_group"] = R;
  t->scalar["sub_rows"] = sub_rows;

  // workgroup trips: BLB runs of about equal cost, in bytes of element stream.  A trip pays for its
  // elements, for every row piece (the LDS access that ends it and its write-back: about as much as
  // four elements) and for one slice copy per slice it enters.
  std::vector<uint64_t> blk_slice(B), blk_rg(B), blk_cost(B);
  const uint64_t elem_bytes = vs + 2 + 1, piece_cost = 4 * elem_bytes, slice_cost = S * vs;
  for (uint64_t b = 0; b < B; b++) {
    blk_slice[b] = col[bl.coo_begin[b]] / S;
    blk_rg[b] = row[bl.coo_begin[b]] / R;
    uint64_t pieces = 1;
    for (uint64_t k = bl.coo_begin[b] + 1; k < bl.coo_begin[b + 1]; k++) pieces += row[k] != row[k - 1];
    blk_cost[b] = (bl.coo_begin[b + 1] - bl.coo_begin[b]) * elem_bytes + pieces * piece_cost;
  }
  // one trip per workgroup the 256 CUs hold at a time with this much LDS each
  uint64_t want = device_facts().cu_num * std::max<uint64_t>(1, device_facts().lds_bytes / ((S + R) * vs));
  want = std::max<uint64_t>(1, std::min<uint64_t>(want, (n + 16383) / 16384));
  std::vector<uint64_t> group_first_block{0};
  // Row ownership (own_rows): the elements are taken row group by row group and a trip is a whole number of row
  // groups, so that one workgroup holds every sum of its rows: the cells of a row group live in LDS across its
  // runs, a cell is the row's place in the group, and at the end of the group the rows are STORED to y -- no
  // atomics, no table of places, y needs no clear.  The price is one copy of x into LDS per run of every row group
  // instead of one per trip and slice, and trips as coarse as row groups: the form is turned down (nullptr) where
  // the copies would move more than a quarter of the element stream's bytes, where there are fewer trips than half
  // the workgroups the device holds, or where the heaviest trip would take more than 1.2 times the average.  It
  // fits matrices of many row groups that meet few slices each (banded matrices); strips of a few very long rows
  // stay with the slice-by-slice order.
  // The runs of the element stream: elements [begin, end) of `order` (row ownership) or of the format's own order,
  // the first column of the stretch of x the run reads, and its row group.
  struct Run { uint64_t begin, end, col0, rg; };
  std::vector<Run> runs;
  std::vector<uint64_t> trip_first_run, trip_first_row_group;
  std::vector<uint32_t> order;  // row ownership: element numbers of the format in the order of the stream
  if (own_rows) {
    if (sub_block_is_col_restricted(m, sub)) return nullptr;  // another sub-matrix adds to the same rows
    AS_CHECK(n < (1ull << 32), "sub-matrix too large for 32-bit element offsets");
    // the rules below, on what is known before anything is re-ordered: there are no more trips than row groups,
    // and a window of x covers at most two slices of the grid, so a row group has at least half as many runs as tiles
    {
      uint64_t tiles = 0, stream = 0;
      for (uint64_t b = 0; b < B; b++) {
        tiles += b == 0 || blk_slice[b] != blk_slice[b - 1] || blk_rg[b] != blk_rg[b - 1];
        stream += blk_cost[b];
      }
      if ((sub_rows + R - 1) / R * 2 < want || (tiles + 1) / 2 * slice_cost * 4 > stream) return nullptr;
    }
    std::vector<uint64_t> blk_order(B);
    for (uint64_t b = 0; b < B; b++) blk_order[b] = b;
    std::stable_sort(blk_order.begin(), blk_order.end(), [&](uint64_t x, uint64_t y) {
      return blk_rg[x] != blk_rg[y] ? blk_rg[x] < blk_rg[y] : blk_slice[x] < blk_slice[y];
    });
    // A row group does not read x slice by slice of the format's grid but window by window: a window starts at the
    // group's first column not yet covered (rounded down to a 16-byte boundary of x) and is col_slice columns wide.
    // The rows of a banded matrix fit one window where they straddle two or three slices of the grid, and a window
    // is one copy of x into LDS and one run.  Inside a window the elements go row by row.
    const uint64_t NG = (sub_rows + R - 1) / R, align = 16 / vs;
    std::vector<uint64_t> group_cost(NG, 0), group_first_own_run(NG + 1, 0);
    uint64_t stream_cost = 0;
    order.reserve(n);
    std::vector<uint32_t> members, sorted;
    std::vector<uint64_t> row_count(R + 1);
    for (uint64_t i = 0; i < B;) {
      const uint64_t g = blk_rg[blk_order[i]];
      members.clear();
      for (; i < B && blk_rg[blk_order[i]] == g; i++) {
        const uint64_t b = blk_order[i];
        group_cost[g] += blk_cost[b];
        for (uint64_t k = bl.coo_begin[b]; k < bl.coo_begin[b + 1]; k++) members.push_back((uint32_t)k);
      }
      stream_cost += group_cost[g];
      group_first_own_run[g] = runs.size();
      for (uint64_t covered = 0;;) {
        uint64_t lo = ~0ull;
        for (uint32_t k : members)
          if (col[k] >= covered && col[k] < lo) lo = col[k];
        if (lo == ~0ull) break;
        const uint64_t w0 = lo / align * align, w1 = w0 + S;
        // the window's elements row by row (a stable counting sort: inside a row the order of the format stays)
        std::fill(row_count.begin(), row_count.end(), 0);
        uint64_t inside = 0;
        for (uint32_t k : members)
          if (col[k] >= covered && col[k] < w1) row_count[row[k] - g * R + 1]++, inside++;
        for (uint64_t r = 0; r < R; r++) row_count[r + 1] += row_count[r];
        sorted.resize(inside);
        for (uint32_t k : members)
          if (col[k] >= covered && col[k] < w1) sorted[row_count[row[k] - g * R]++] = k;
        runs.push_back({order.size(), order.size() + inside, w0, g});
        order.insert(order.end(), sorted.begin(), sorted.end());
        group_cost[g] += slice_cost;
        covered = w1;
      }
    }
    group_first_own_run[NG] = runs.size();
    // A row group without elements has no run: the workgroup that owns it never reaches the group's stores, and
    // its rows of y are then written by nobody (template_needs_cleared_y asks for the clear of y)
    uint64_t groups_without_run = 0;
    for (uint64_t g = NG; g-- > 0;)
      if (group_cost[g] == 0) {
        group_first_own_run[g] = group_first_own_run[g + 1];
        groups_without_run++;
      }
    t->scalar["row_groups_without_elements"] = groups_without_run;
    if (runs.size() * slice_cost * 4 > stream_cost) return nullptr;
    uint64_t total = 0;
    for (uint64_t c : group_cost) total += c;
    // as many trips as workgroups fit, or the fewest more row groups per trip that make the trips even
    const uint64_t groups_per_trip = (NG + want - 1) / want;
    const uint64_t trips = (NG + groups_per_trip - 1) / groups_per_trip, per_trip = total / trips + 1;
    uint64_t cost = 0, heaviest = 0;
    trip_first_row_group.push_back(0);
    for (uint64_t g = 0; g < NG; g++) {
      if (cost > 0 && cost + group_cost[g] / 2 > per_trip && trip_first_row_group.size() < trips) {
        heaviest = std::max(heaviest, cost);
        trip_first_row_group.push_back(g);
        cost = 0;
      }
      cost += group_cost[g];
    }
    heaviest = std::max(heaviest, cost);
    trip_first_row_group.push_back(NG);
    const uint64_t T = trip_first_row_group.size() - 1;
    // too few trips leave most CUs idle; uneven trips make the others wait for the heaviest
    if (T * 2 < want || heaviest * T * 10 > total * 12) return nullptr;
    for (uint64_t tp = 0; tp <= T; tp++) trip_first_run.push_back(group_first_own_run[trip_first_row_group[tp]]);
  } else {
  uint64_t total_cost = want * slice_cost;
  for (uint64_t b = 0; b < B; b++) {
    total_cost += blk_cost[b];
    if (b == 0 || blk_slice[b] != blk_slice[b - 1]) total_cost += slice_cost;
  }
  // Greedy cuts at a cost of `per_group` each.  The cuts fall between BLBs, so a trip may end short of its share and
  // the count can come out a few above `want` -- with one workgroup per CU those few would wait for a second round
  // and the kernel would take nearly twice as long (measured: 259 trips 54.3 us, 247 trips 33.7 us on the same
  // strip).  The share is raised until the trips fit.
  uint64_t per_group = total_cost / want + 1;
  for (;;) {
    group_first_block.assign(1, 0);
    uint64_t cost = 0;
    for (uint64_t b = 0; b < B; b++) {
      bool first = group_first_block.back() == b;
      uint64_t c = blk_cost[b];
      if (first || blk_slice[b] != blk_slice[b - 1]) c += slice_cost;
      if (!first && cost + c / 2 > per_group) {
        group_first_block.push_back(b);
        cost = 0;
        c = blk_cost[b] + slice_cost;
      }
      cost += c;
    }
    group_first_block.push_back(B);
    if (group_first_block.size() - 1 <= want) break;
    per_group += per_group / 64 + 1;
  }
  // runs: maximal sequences of BLBs of one tile inside a trip
  for (uint64_t g = 0; g + 1 < group_first_block.size(); g++) {
    trip_first_run.push_back(runs.size());
    for (uint64_t b = group_first_block[g], e; b < group_first_block[g + 1]; b = e) {
      for (e = b + 1; e < group_first_block[g + 1] && blk_slice[e] == blk_slice[b] && blk_rg[e] == blk_rg[b];) e++;
      runs.push_back({bl.coo_begin[b], bl.coo_begin[e], blk_slice[b] * S, blk_rg[b]});
    }
  }
  trip_first_run.push_back(runs.size());
  }
  const uint64_t G = trip_first_run.size() - 1;
  t->scalar["group_num"] = G;
  t->own_rows = own_rows;

  // y row of every row of the sub-matrix (through the sort permutation when there is one)
  std::vector<uint64_t> y_row(sub_rows);
  for (uint64_t r = 0; r < sub_rows; r++) y_row[r] = r;
  t->global_sort_index = apply_global_sort(m, sub, y_row, sub_rows);
  // A sort permutation scatters the strip's rows over all of y, and an atomic on a line no other
  // row of the strip touches costs a trip to memory.  The sums are then collected in a dense
  // scratch vector (one value per row of the strip) and moved to y by spmv_<sub>_finish, with plain
  // stores: the rows of a row strip belong to this kernel alone.
  if (own_rows) {
    t->is_atom_add = false;  // every row is stored once, by the workgroup that owns its row group
  } else if (t->global_sort_index && !sub_block_is_col_restricted(m, sub)) {
    t->scratch_bytes = sub_rows * vs;
    t->scratch_starts_zero = true;  // row sums are added into it; the finish kernel leaves it cleared
    t->is_atom_add = false;  // y itself is written once, by the finish kernel
    t->finish_tblock_num = std::max<uint64_t>(1, std::min<uint64_t>(1024, (sub_rows + 255) / 256));
  }
  // where the write-back of a piece goes: the row's cell of the scratch vector, or its row of y
  const uint64_t y_base = !t->global_sort_index ? t->kernal_first_row_index : 0;
  auto target_of = [&](uint64_t sub_row) { return t->scratch_bytes ? sub_row : y_row[sub_row] + y_base; };

  // runs: maximal sequences of BLBs of one tile inside a trip, padded to kRunUnit elements.  A piece is numbered
  // by its order inside the run -- or, under row ownership, by the row's place in its row group, which every run
  // of the group shares; a lane's pieces must then still be consecutive numbers, so where a row of the group has
  // no element in the slice the lane is closed with zero-valued elements and the next row opens a new lane.
  std::vector<uint64_t> group_first_run, run_slice, run_nz_begin{0}, run_piece_begin{0}, piece_target, run_row_group;
  std::vector<uint64_t> lcol, piece;  // per element: column inside the slice, piece number inside the run
  uint64_t lane_runs = 0;             // column-run form: runs of consecutive columns in the lane being filled
  lcol.reserve(n + G * kRunUnit);
  piece.reserve(n + G * kRunUnit);
  t->val_arr.reserve(n + G * kRunUnit);
  auto elem = [&](uint64_t i) { return own_rows ? (uint64_t)order[i] : i; };
  std::vector<ValVec> other_rows(row_block - 1);  // row blocks: the values of rows 1 .. b-1 of every element
  for (uint64_t g = 0; g < G; g++) {
    group_first_run.push_back(run_slice.size());
    for (uint64_t ri = trip_first_run[g]; ri < trip_first_run[g + 1]; ri++) {
      const Run &run = runs[ri];
      const uint64_t col0 = run.col0, row0 = run.rg * R;
      const uint64_t slice_len = std::min<uint64_t>(S, t->matrix_cols - t->kernal_first_col_index - col0);
      uint64_t pieces = 0, cur_piece = 0;
      // a zero-valued element on the current piece; in the column-run form its column continues the run where
      // that stays inside the slice, and otherwise opens a run at column 0
      auto pad = [&]() {
        uint64_t c = 0;
        if (column_runs && lcol.size() % kLaneElems != 0 && lcol.back() + 1 < slice_len) c = lcol.back() + 1;
        else if (column_runs) lane_runs++;
        lcol.push_back(c);
        piece.push_back(cur_piece);
        t->val_arr.push_back(0.0);
      };
      // one step of the loop = one element of the stream: an element of a row, or (row blocks) the elements that
      // the rows of a block hold in one column
      uint64_t prev_row = 0;   // first row of the piece before
      auto take = [&](uint64_t k, uint64_t piece_row, bool first, bool new_row) {
        const uint64_t c = col[k] - col0;
        // row ownership: a row that does not follow its predecessor directly cannot share a lane with it
        if (own_rows && new_row && !first && piece_row != prev_row + row_block)
          while (lcol.size() % kLaneElems) pad();
        if (column_runs) {
          if (lcol.size() % kLaneElems == 0) lane_runs = 0;
          if (lcol.size() % kLaneElems == 0 || c != lcol.back() + 1) {
            if (lane_runs >= kLaneRuns) {
              while (lcol.size() % kLaneElems) pad();   // pieces >= 1 here: the lane holds elements of this run
              lane_runs = 0;
            }
            lane_runs++;
          }
        }
        if (new_row) {
          if (!own_rows) piece_target.push_back(target_of(piece_row));
          pieces++;
          cur_piece = own_rows ? piece_row - row0 : pieces - 1;
          prev_row = piece_row;
        }
        lcol.push_back(c);
        piece.push_back(cur_piece);
        t->val_arr.push_back(val[k]);
      };
      if (row_block == 1) {
        for (uint64_t i = run.begin; i < run.end; i++) {
          const uint64_t k = elem(i);
          const bool first = i == run.begin;
          take(k, row[k], first, first || row[k] != row[elem(i - 1)]);
        }
      } else {
        for (uint64_t i = run.begin; i < run.end;) {
          const uint64_t r0 = row[elem(i)];
          if (r0 % row_block != 0 || r0 + row_block > sub_rows) return nullptr;  // the block's first row is missing here
          uint64_t first_of[5];
          first_of[0] = i;
          for (uint64_t q = 0; q < row_block; q++) {
            uint64_t j = first_of[q];
            while (j < run.end && row[elem(j)] == r0 + q) j++;
            first_of[q + 1] = j;
          }
          const uint64_t len = first_of[1] - first_of[0];
          for (uint64_t q = 1; q < row_block; q++) {
            if (first_of[q + 1] - first_of[q] != len) return nullptr;
            for (uint64_t e = 0; e < len; e++)
              if (col[elem(first_of[q] + e)] != col[elem(first_of[0] + e)]) return nullptr;
          }
          for (uint64_t e = 0; e < len; e++) {
            take(elem(first_of[0] + e), r0, i == run.begin && e == 0, e == 0);
            // the other rows' values of this element, in planes of their own until the stream is laid out
            for (uint64_t q = 1; q < row_block; q++) {
              other_rows[q - 1].resize(t->val_arr.size() - 1, 0.0);
              other_rows[q - 1].push_back(val[elem(first_of[q] + e)]);
            }
          }
          i = first_of[row_block];
        }
      }
      AS_CHECK(pieces <= R && cur_piece < R, "more row pieces in a run than rows in a row group");
      while (lcol.size() % kRunUnit) {
        if (column_runs && lcol.size() % kLaneElems == 0) lane_runs = 0;
        pad();
      }
      run_slice.push_back(own_rows ? col0 : col0 / S);
      run_row_group.push_back(run.rg);
      run_nz_begin.push_back(lcol.size() / kRunUnit);
      run_piece_begin.push_back(piece_target.size());
    }
  }
  group_first_run.push_back(run_slice.size());
  const uint64_t padded = lcol.size();
  AS_CHECK(padded < (1ull << 32) && piece_target.size() < (1ull << 32), "sub-matrix too large for 32-bit element offsets");

  // Lane words.  The kernel emits a sum where a piece ends inside a lane's elements, and at the last lane of
  // every stretch of lanes whose last elements share a piece (the wave-wide segmented sum).  Most short
  // pieces get exactly one such sum before the run's write-back: those are marked, and the kernel stores
  // them into the piece's LDS cell instead of adding atomically -- LDS atomics are the slower by far.
  std::vector<uint64_t> lane_word(padded / kLaneElems, 0);
  {
    std::vector<uint32_t> sums_of_piece;
    auto for_each_sum = [&](uint64_t p0, uint64_t p1, auto &&f) {
      for (uint64_t u = p0; u < p1; u += kRunUnit)
        for (uint64_t lane = 0; lane < 64; lane++) {
          const uint64_t at = u + kLaneElems * lane, last = at + kLaneElems - 1;
          for (uint64_t j = 0; j + 1 < kLaneElems; j++)
            if (piece[at + j] != piece[at + j + 1]) f(at + j);
          if (lane == 63 || piece[last] != piece[last + kLaneElems]) f(last);
        }
    };
    for (uint64_t run = 0; run < run_slice.size(); run++) {
      const uint64_t p0 = run_nz_begin[run] * kRunUnit, p1 = run_nz_begin[run + 1] * kRunUnit;
      sums_of_piece.assign(own_rows ? R : run_piece_begin[run + 1] - run_piece_begin[run], 0);
      for (uint64_t at = p0; at < p1; at += kLaneElems) {
        uint64_t w = piece[at];
        for (uint64_t j = 1; j < kLaneElems; j++) {
          AS_CHECK(piece[at + j] == piece[at + j - 1] || piece[at + j] == piece[at + j - 1] + row_block, "pieces must be consecutive");
          if (piece[at + j] != piece[at + j - 1]) w |= 1ull << (kNewPieceBit + j);
        }
        lane_word[at / kLaneElems] = w;
      }
      for_each_sum(p0, p1, [&](uint64_t at) { sums_of_piece[piece[at]]++; });
      for_each_sum(p0, p1, [&](uint64_t at) {
        if (sums_of_piece[piece[at]] == 1) lane_word[at / kLaneElems] |= 1ull << (kStoreBit + at % kLaneElems);
      });
    }
  }
  std::vector<uint64_t> col_run_mask;
  if (column_runs) {
    // per lane the first column of its first kLaneRuns runs, and the byte of run starts (bit j: element j opens
    // the next run); a start beyond those decodes as column 0, and only padding opens such a run
    std::vector<uint64_t> starts(padded / kLaneElems * kLaneRuns, 0);
    col_run_mask.assign(padded / kLaneElems, 0);
    for (uint64_t at = 0; at < padded; at += kLaneElems) {
      unsigned runs = 0;
      for (uint64_t j = 0; j < kLaneElems; j++) {
        if (j != 0 && lcol[at + j] == lcol[at + j - 1] + 1) continue;
        if (j != 0) col_run_mask[at / kLaneElems] |= 1ull << j;
        if (runs < kLaneRuns) starts[at / kLaneElems * kLaneRuns + runs] = lcol[at + j];
        else AS_CHECK(lcol[at + j] == 0, "a lane holds more column runs than it has room for");
        runs++;
      }
    }
    lcol.swap(starts);
    t->col_runs = true;
  }
  t->col_index_arr.assign(std::move(lcol), UNSIGNED_SHORT);
  // Values are read 16 bytes per lane and load; for the 64 lanes of a load to read one contiguous kilobyte,
  // the 16-byte pieces of a wavefront step are stored load by load: piece i of lane l at (i * 64 + l).
  // Row blocks: the b rows of a lane one after the other, each in its 16-byte pieces.
  {
    const uint64_t chunk = 16 / vs, chunks = kLaneElems / chunk, b = row_block;
    for (ValVec &plane : other_rows) plane.resize(padded, 0.0);
    ValVec stored(padded * b);
    for (uint64_t u = 0; u < padded; u += kRunUnit)
      for (uint64_t lane = 0; lane < 64; lane++)
        for (uint64_t q = 0; q < b; q++) {
          const ValVec &plane = q == 0 ? t->val_arr : other_rows[q - 1];
          for (uint64_t j = 0; j < kLaneElems; j++)
            stored[u * b + ((q * chunks + j / chunk) * 64 + lane) * chunk + j % chunk] = plane[u + lane * kLaneElems + j];
        }
    t->val_arr.swap(stored);
    std::vector<ValVec>().swap(other_rows);
  }
  t->scalar["row_block"] = row_block;
  t->row_block = row_block;

  // the run tables are read with scalar loads, which need 32-bit entries
  auto add = [&](const char *name, std::vector<uint64_t> v, bool word) {
    TArr a;
    a.name = name;
    uint64_t mx = v.empty() ? 0 : *std::max_element(v.begin(), v.end());
    a.a.assign(std::move(v), word && mx <= 0xffffffffull ? UNSIGNED_INT : suitable_dtype(mx));
    t->arrays.push_back(std::move(a));
  };
  add("group_first_run", std::move(group_first_run), true);
  add(own_rows ? "run_col_begin" : "run_slice", std::move(run_slice), true);
  add("run_nz_begin", std::move(run_nz_begin), true);
  if (own_rows) {
    add("run_row_group", std::move(run_row_group), true);
  } else {
    add("run_piece_begin", std::move(run_piece_begin), true);
    add("piece_target", std::move(piece_target), true);
  }
  add("lane_word", std::move(lane_word), true);
  if (column_runs) {
    TArr a;
    a.name = "col_run_mask";
    a.a.assign(std::move(col_run_mask), UNSIGNED_CHAR);
    t->arrays.push_back(std::move(a));
  }
  add("y_row_index", std::move(y_row), false);
  // the finish kernel's map (the main kernel has piece_target), or the map of the rows a workgroup owns
  t->find("y_row_index")->on_device = t->finish_tblock_num != 0 || (own_rows && t->global_sort_index);
  if (own_rows) {
    add("trip_first_row_group", std::move(trip_first_row_group), false);  // host only
    t->find("trip_first_row_group")->on_device = false;
  } else {
    add("group_first_block", std::move(group_first_block), false);  // BLB view of the trips, host only
    t->find("group_first_block")->on_device = false;
  }
  tpl_shared_memory_tile::set_default_launch(*t);
  return t;
}

void try_all_compress(Template &t) {
  for (const char *name : {"group_first_run", "run_slice", "run_col_begin", "run_nz_begin", "run_piece_begin", "run_row_group", "y_row_index"}) {
    TArr *a = t.find(name);
    if (a && !a->c.active()) init_linear_compressor(a->a, a->c, true);
  }
}

void set_default_launch(Template &t) {
  if (t.thread_num_in_block == 0) t.thread_num_in_block = 1024;
  t.tblock_num = std::max<uint64_t>(1, std::min<uint64_t>(t.sc("group_num"), (1ull << 31) - 1));
  t.dynamic_lds_bytes = (t.sc("col_slice") + t.sc("row_group")) * (uint64_t)dtype_size(t.val_dtype);
}

std::string kernel_source(const Template &t) {
  const std::string vt = value_type_name(t);
  AS_CHECK(t.col_index_arr.dt == UNSIGNED_SHORT && t.arr("lane_word").a.dt == UNSIGNED_INT &&
               (t.own_rows || t.arr("piece_target").a.dt == UNSIGNED_INT),
           "slice columns must be 16 bits wide, lane words and piece targets 32");
  AS_CHECK(t.thread_num_in_block % 64 == 0 && t.thread_num_in_block >= 64 && t.thread_num_in_block <= 1024,
           "thread_num_in_block must be a multiple of 64 up to 1024");
  const uint64_t S = t.sc("col_slice"), R = t.sc("row_group"), G = t.sc("group_num"), rows = t.sc("sub_rows");
  const std::string id = std::to_string(t.sub), B = std::to_string(t.thread_num_in_block) + "u";
  const std::string Ss = std::to_string(S) + "u", Rs = std::to_string(R) + "u", Ks = std::to_string(kBatch);
  const std::string Ls = std::to_string(kLaneElems), Us = std::to_string(kRunUnit) + "u";
  // x is read from kernal_first_col_index on; columns of the sub-matrix are relative to it
  const uint64_t x_len = t.matrix_cols - t.kernal_first_col_index;
  const bool wide_copy = t.kernal_first_col_index % 4 == 0;
  const std::string target = t.scratch_bytes ? "(" + vt + " *)scratch_arr" : "device_y_arr";
  std::string s;
  // The body is a device function of its own: the kernel spmv_<id> runs it for its own workgroups, and the first
  // kernel of the strip behind this one can run it ahead of its own trips (Template::fused_trips).  as_block /
  // as_grid: the number of the workgroup among those that run the trips, and how many they are.
  // (C linkage like the kernels: the declaration of the dynamic LDS array inside it must agree with theirs)
  s += "extern \"C\" __device__ __forceinline__ void " + kernel_trips_function_name(t) + "(" + kernel_signature(t) +
       ", const unsigned int as_block, const unsigned int as_grid)\n{\n";
  // row blocks: a lane's loads of values cover its eight elements in each of the block's rows
  const unsigned RB = t.scalar.count("row_block") ? (unsigned)t.sc("row_block") : 1u;
  const unsigned chunk = 16 / (unsigned)dtype_size(t.val_dtype), chunks = (unsigned)kLaneElems / chunk;
  const std::string Cs = std::to_string(chunk), Ns = std::to_string(chunks * RB);
  s += "  typedef " + vt + " val16_t __attribute__((ext_vector_type(" + Cs + ")));\n";  // 16 bytes of values
  if (t.col_runs) {
    AS_CHECK(t.arr("col_run_mask").a.dt == UNSIGNED_CHAR, "run masks must be bytes");
    s += "  typedef unsigned long long col8_t;\n";  // the first columns of four runs, 16 bits each
  } else {
    s += "  typedef unsigned short col8_t __attribute__((ext_vector_type(8)));\n";
  }
  s += "  extern __shared__ __attribute__((aligned(16))) unsigned char as_dynamic_lds[];\n";
  s += "  " + vt + " *x_slice = (" + vt + " *)as_dynamic_lds;\n";
  s += "  " + vt + " *piece_sum = x_slice + " + Ss + ";\n";
  // the wavefront's number and the run bounds are the same in all lanes: kept in scalar registers, they make the
  // table reads scalar loads and the loop branches scalar branches
  s += "  const unsigned int lane = threadIdx.x & 63u, wave_in_block = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);\n";
  s += "  const unsigned int stride = (" + B + " >> 6) * " + Us + ";\n";
  s += "  const " + vt + " *x_sub = device_x_arr + " + std::to_string(t.kernal_first_col_index) + "u;\n";
  s += "  for (unsigned int grp = as_xcd_block_index(as_block, as_grid); grp < " + std::to_string(G) + "u; grp += as_grid)\n  {\n";
  s += "    unsigned int next_grp = grp + 1u, run_begin, run_end;\n";
  s += "    " + code_of_meta_read(t, "group_first_run", "run_begin", "grp");
  s += "    " + code_of_meta_read(t, "group_first_run", "run_end", "next_grp");
  s += "    run_begin = __builtin_amdgcn_readfirstlane(run_begin); run_end = __builtin_amdgcn_readfirstlane(run_end);\n";
  s += "    as_barrier();\n";  // the previous trip's write-back is done with the cells
  s += "    for (unsigned int i = threadIdx.x; i < " + Rs + "; i += " + B + ") piece_sum[i] = 0;\n";
  if (t.own_rows) s += "    unsigned int cur_slice = 0xffffffffu, cur_group = 0xffffffffu;\n";
  else s += "    unsigned int cur_slice = 0xffffffffu, done_begin = 0u, done_end = 0u;\n";
  s += "    for (unsigned int run = run_begin; run <= run_end; run++)\n    {\n";
  // run == run_end is the write-back of the trip's last run
  s += "      unsigned int next_run = run + 1u, slice = 0xffffffffu, unit_begin = 0u, unit_end = 0u, piece_begin = 0u, piece_end = 0u, row_group = 0xffffffffu;\n";
  s += "      if (run < run_end)\n      {\n";
  s += "        " + code_of_meta_read(t, t.own_rows ? "run_col_begin" : "run_slice", "slice", "run");
  s += "        " + code_of_meta_read(t, "run_nz_begin", "unit_begin", "run");
  s += "        " + code_of_meta_read(t, "run_nz_begin", "unit_end", "next_run");
  if (t.own_rows) {
    s += "        " + code_of_meta_read(t, "run_row_group", "row_group", "run");
  } else {
    s += "        " + code_of_meta_read(t, "run_piece_begin", "piece_begin", "run");
    s += "        " + code_of_meta_read(t, "run_piece_begin", "piece_end", "next_run");
  }
  s += "      }\n";
  s += "      as_barrier();\n";  // every wavefront is done with the previous run
  // Between two runs a workgroup writes the finished run back (a table read and one atomic per piece) and, when the
  // slice changes, copies the new slice of x into LDS.  Written as plain loops, both are chains of memory round
  // trips: the compiler waits for an atomic to complete before it lets anything overwrite the atomic's data
  // registers, and for each load of the copy before its LDS store, so every iteration costs a trip (or two) to
  // memory.  Here a lane first requests everything it needs -- the sums, the places and the addresses of its
  // pieces -- then issues its atomics back to back from registers nobody writes in between; the slice copy
  // requests a batch of loads before it stores the first.
  const uint64_t wb_batch = std::min<uint64_t>(kBetweenRunsBatch, std::max<uint64_t>(1, (R + t.thread_num_in_block - 1) / t.thread_num_in_block));
  const std::string Ws = std::to_string(wb_batch);
  if (t.own_rows) {
    // Row ownership: a row group's cells stay in LDS across its runs (one per slice it meets); when the coming run
    // belongs to another row group -- or the trip ends -- the finished group's rows are stored to y, zeros for rows
    // without elements included: no other workgroup holds a sum of these rows.
    const std::string y_off = (!t.global_sort_index && t.kernal_first_row_index != 0 ? " + " + std::to_string(t.kernal_first_row_index) + "u" : std::string());
    s += "      if (row_group != cur_group)\n      {\n";
    s += "        if (cur_group != 0xffffffffu)\n        {\n";
    s += "          const unsigned int row0 = cur_group * " + Rs + ", live = min(" + Rs + ", " + std::to_string(rows) + "u - row0);\n";
    s += "          for (unsigned int i = threadIdx.x; i < live; i += " + B + ")\n          {\n";
    s += "            const " + vt + " sum = piece_sum[i];\n            piece_sum[i] = 0;\n";
    s += "            const unsigned int sub_row = row0 + i;\n            unsigned int global_row_index;\n";
    if (t.global_sort_index) s += "            " + code_of_meta_read(t, "y_row_index", "global_row_index", "sub_row");
    else s += "            global_row_index = sub_row;\n";
    s += "            as_stnt(device_y_arr + global_row_index" + y_off + ", sum);\n";
    s += "          }\n        }\n";
    s += "        cur_group = row_group;\n      }\n";
  } else {
  // write-back of the run that ended: consecutive lanes take consecutive pieces (rows in rising order)
  s += "      for (unsigned int i0 = threadIdx.x; i0 < done_end - done_begin; i0 += " + B + " * " + Ws + "u)\n      {\n";
  s += "        typedef __attribute__((address_space(1))) " + vt + " *global_ptr_t;\n";
  s += "        " + vt + " sum[" + Ws + "];\n        unsigned int place[" + Ws + "];\n        global_ptr_t where[" + Ws + "];\n";
  s += "        #pragma unroll\n        for (int j = 0; j < " + Ws + "; j++)\n        {\n";
  s += "          const unsigned int i = i0 + j * " + B + ";\n";
  s += "          sum[j] = 0;\n          place[j] = 0u;\n";
  s += "          if (i < done_end - done_begin)\n          {\n";
  s += "            sum[j] = piece_sum[i];\n            piece_sum[i] = 0;\n";
  s += "            const unsigned int at = done_begin + i;\n";
  s += "            " + code_of_meta_read(t, "piece_target", "place[j]", "at");
  s += "          }\n        }\n";
  // (the empty asm pins every address in registers of its own here, ahead of the atomics)
  s += "        #pragma unroll\n        for (int j = 0; j < " + Ws + "; j++)\n        {\n          where[j] = (global_ptr_t)(" + target + " + place[j]);\n          asm volatile(\"\" : \"+v\"(where[j]));\n        }\n";
  s += "        __builtin_amdgcn_sched_barrier(0);\n";  // every address is in its registers before the first atomic goes out
  s += "        #pragma unroll\n        for (int j = 0; j < " + Ws + "; j++)\n";
  s += "          if (sum[j] != 0) __builtin_amdgcn_global_atomic_fadd_" + std::string(t.val_dtype == DOUBLE ? "f64" : "f32") + "(where[j], sum[j]);\n";
  s += "      }\n";
  s += "      done_begin = piece_begin; done_end = piece_end;\n";
  }
  s += "      if (run < run_end && slice != cur_slice)\n      {\n";
  // under row ownership the table holds the first column of the run's stretch of x itself
  s += "        const unsigned int col0 = slice" + (t.own_rows ? std::string() : " * " + Ss) + ";\n";
  s += "        const unsigned int slice_len = min(" + Ss + ", " + std::to_string(x_len) + "u - col0);\n";
  const std::string Ks2 = std::to_string(kBetweenRunsBatch);
  if (wide_copy) {
    // 16 bytes per lane and load: the 64 lanes of a load read one contiguous kilobyte
    s += "        for (unsigned int i0 = threadIdx.x * " + Cs + "u; i0 + " + Cs + "u <= slice_len; i0 += " + Ks2 + "u * " + B + " * " + Cs + "u)\n        {\n";
    s += "          val16_t part[" + Ks2 + "];\n";
    s += "          #pragma unroll\n          for (int j = 0; j < " + Ks2 + "; j++)\n";
    s += "            if (i0 + j * " + B + " * " + Cs + "u + " + Cs + "u <= slice_len) part[j] = *(const val16_t *)(x_sub + col0 + i0 + j * " + B + " * " + Cs + "u);\n";
    s += "          #pragma unroll\n          for (int j = 0; j < " + Ks2 + "; j++)\n";
    s += "            if (i0 + j * " + B + " * " + Cs + "u + " + Cs + "u <= slice_len) *(val16_t *)(x_slice + i0 + j * " + B + " * " + Cs + "u) = part[j];\n";
    s += "        }\n";
    s += "        if (threadIdx.x < slice_len % " + Cs + "u) x_slice[slice_len / " + Cs + "u * " + Cs + "u + threadIdx.x] = x_sub[col0 + slice_len / " + Cs + "u * " + Cs + "u + threadIdx.x];\n";
  } else {
    s += "        for (unsigned int i0 = threadIdx.x; i0 < slice_len; i0 += " + Ks2 + "u * " + B + ")\n        {\n";
    s += "          " + vt + " one[" + Ks2 + "];\n";
    s += "          #pragma unroll\n          for (int j = 0; j < " + Ks2 + "; j++)\n";
    s += "            if (i0 + j * " + B + " < slice_len) one[j] = x_sub[col0 + i0 + j * " + B + "];\n";
    s += "          #pragma unroll\n          for (int j = 0; j < " + Ks2 + "; j++)\n";
    s += "            if (i0 + j * " + B + " < slice_len) x_slice[i0 + j * " + B + "] = one[j];\n";
    s += "        }\n";
  }
  s += "        cur_slice = slice;\n      }\n";
  s += "      as_barrier();\n";
  // Runs are padded to whole wavefront steps: a step is inside the run for all lanes or for none, and the steps
  // outside are neither loaded nor used.  All loads of a full batch are requested before the first is used.
  auto load_step = [&](const std::string &ind) {
    std::string c;
    c += ind + "const unsigned int unit = nz0 + k * stride, at = unit + lane * " + Ls + "u;\n";
    c += ind + "#pragma unroll\n";
    c += ind + "for (int i = 0; i < " + Ns + "; i++) a[k][i] = as_ldnt((const val16_t *)(val_arr + unit" + (RB > 1 ? " * " + std::to_string(RB) + "u" : std::string()) + " + (i * 64u + lane) * " + Cs + "u));\n";
    if (t.col_runs) {
      c += ind + "c[k] = as_ldnt((const col8_t *)(col_index_arr + (at >> 1)));\n";
      c += ind + "m[k] = as_ldnt(col_run_mask + (at >> 3));\n";
    } else {
      c += ind + "c[k] = as_ldnt((const col8_t *)(col_index_arr + at));\n";
    }
    c += ind + "w[k] = as_ldnt(lane_word + (at >> 3));\n";
    return c;
  };
  s += "      const unsigned int nz_end = unit_end * " + Us + ";\n";
  s += "      for (unsigned int nz0 = unit_begin * " + Us + " + wave_in_block * " + Us + "; nz0 < nz_end; nz0 += stride * " + Ks + "u)\n      {\n";
  s += "        val16_t a[" + Ks + "][" + Ns + "];\n        col8_t c[" + Ks + "];\n        unsigned int w[" + Ks + "];\n";
  if (t.col_runs) s += "        unsigned char m[" + Ks + "];\n";
  s += "        if (nz0 + (" + Ks + "u - 1u) * stride < nz_end)\n        {\n";
  s += "          #pragma unroll\n          for (int k = 0; k < " + Ks + "; k++)\n          {\n" + load_step("            ") + "          }\n";
  s += "        }\n        else\n        {\n";
  s += "          #pragma unroll\n          for (int k = 0; k < " + Ks + " - 1; k++)\n          {\n";
  s += "            if (nz0 + k * stride < nz_end)\n            {\n" + load_step("              ") + "            }\n          }\n        }\n";
  s += "        #pragma unroll\n        for (int k = 0; k < " + Ks + "; k++)\n        {\n";
  s += "          if (nz0 + k * stride >= nz_end) break;\n";
  // the eight x values are requested together, ahead of the sums that may touch LDS in between
  s += "          " + vt + " xv[" + Ls + "];\n";
  if (t.col_runs) {
    // element j takes the next run's first column where its bit is set (the starts shift down; past the fourth
    // they are 0), and otherwise the column after the previous element's
    s += "          {\n            unsigned long long starts = c[k];\n            unsigned int col = (unsigned int)starts & 0xffffu;\n";
    s += "            xv[0] = x_slice[col];\n";
    s += "            #pragma unroll\n            for (int j = 1; j < " + Ls + "; j++)\n            {\n";
    s += "              const bool next_run = (m[k] >> j) & 1u;\n";
    s += "              starts >>= next_run ? 16 : 0;\n";
    s += "              col = next_run ? (unsigned int)starts & 0xffffu : col + 1u;\n";
    s += "              xv[j] = x_slice[col];\n            }\n          }\n";
  } else {
    s += "          #pragma unroll\n          for (int j = 0; j < " + Ls + "; j++) xv[j] = x_slice[(unsigned int)c[k][j]];\n";
  }
  // A piece that ends inside the lane is emitted at once; the lane's last piece joins the scan.  A marked sum
  // is the only one of its piece before the write-back: a plain store will do.
  auto emit = [&](unsigned j) {
    const std::string bit = std::to_string(1u << (kStoreBit + j)) + "u";
    // under row ownership a cell may hold the row's sum from an earlier slice: the only sum of its piece IN THIS
    // RUN is added without an atomic (nobody else touches the cell before the next barrier)
    if (RB == 1)
      return "{ if (w[k] & " + bit + ") piece_sum[cell] " + std::string(t.own_rows ? "+=" : "=") + " acc; else as_lds_add(piece_sum + cell, acc); }";
    // row blocks: the block's rows are neighbouring cells
    std::string plain, atomic;
    for (unsigned q = 0; q < RB; q++) {
      plain += " piece_sum[cell + " + std::to_string(q) + "u] += acc" + std::to_string(q) + ";";
      atomic += " as_lds_add(piece_sum + cell + " + std::to_string(q) + "u, acc" + std::to_string(q) + ");";
    }
    return "{ if (w[k] & " + bit + ") {" + plain + " } else {" + atomic + " } }";
  };
  s += "          unsigned int cell = w[k] & 0x7fffu;\n";
  if (RB == 1) {
    s += "          " + vt + " acc = a[k][0][0] * xv[0];\n";
    for (unsigned j = 1; j < kLaneElems; j++) {
      s += "          if (w[k] & " + std::to_string(1u << (kNewPieceBit + j)) + "u) { " + emit(j - 1) + " acc = 0; cell++; }\n";
      s += "          acc += a[k][" + std::to_string(j / chunk) + "][" + std::to_string(j % chunk) + "] * xv[" + std::to_string(j) + "];\n";
    }
    s += "          acc = as_wave_segmented_sum(cell, acc);\n";
    s += "          if (as_is_segment_tail(cell)) " + emit(kLaneElems - 1) + "\n";
  } else {
    auto value = [&](unsigned q, unsigned j) {
      return "a[k][" + std::to_string(q * chunks + j / chunk) + "][" + std::to_string(j % chunk) + "]";
    };
    for (unsigned q = 0; q < RB; q++)
      s += "          " + vt + " acc" + std::to_string(q) + " = " + value(q, 0) + " * xv[0];\n";
    for (unsigned j = 1; j < kLaneElems; j++) {
      std::string zero;
      for (unsigned q = 0; q < RB; q++) zero += " acc" + std::to_string(q) + " = 0;";
      s += "          if (w[k] & " + std::to_string(1u << (kNewPieceBit + j)) + "u) { " + emit(j - 1) + zero + " cell += " + std::to_string(RB) + "u; }\n";
      for (unsigned q = 0; q < RB; q++)
        s += "          acc" + std::to_string(q) + " += " + value(q, j) + " * xv[" + std::to_string(j) + "];\n";
    }
    for (unsigned q = 0; q < RB; q++)
      s += "          acc" + std::to_string(q) + " = as_wave_segmented_sum(cell, acc" + std::to_string(q) + ");\n";
    s += "          if (as_is_segment_tail(cell)) " + emit(kLaneElems - 1) + "\n";
  }
  s += "        }\n      }\n    }\n  }\n}\n";
  s += "extern \"C\" __global__ void __launch_bounds__(" + std::to_string(t.thread_num_in_block) + ") spmv_" + id + "(" +
       kernel_signature(t) + ")\n{\n  " + kernel_trips_function_name(t) + "(" + kernel_arguments(t, "") + ", blockIdx.x, gridDim.x);\n}\n";
  if (t.finish_tblock_num) {
    s += "extern \"C\" __global__ void __launch_bounds__(256) spmv_" + id + "_finish(" + kernel_signature(t) + ")\n{\n";
    s += "  " + vt + " *row_sum = (" + vt + " *)scratch_arr;\n";
    s += "  for (unsigned int sub_row = blockIdx.x * 256u + threadIdx.x; sub_row < " + std::to_string(rows) +
         "u; sub_row += gridDim.x * 256u)\n  {\n";
    s += "    const " + vt + " sum = row_sum[sub_row];\n";
    s += "    row_sum[sub_row] = 0;\n";
    s += "    unsigned int global_row_index;\n";
    s += "    " + code_of_meta_read(t, "y_row_index", "global_row_index", "sub_row");
    s += "    as_stnt(device_y_arr + global_row_index, sum);\n";
    s += "  }\n}\n";
  }
  return s;
}

}  // namespace tpl_shared_memory_tile
}  // namespace asx
