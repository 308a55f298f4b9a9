// COO input, validation, deep copy.  Host side of rows a1-a3 of the hot path.
#include "matrix.hpp"

#include <cctype>
#include <cstdlib>
#include <cstring>
#include <fstream>

namespace asx {

const char *dtype_name(DType t) {
  static const char *n[] = {"CHAR", "UNSIGNED_CHAR", "SHORT", "UNSIGNED_SHORT", "INT", "UNSIGNED_INT",
                            "LONG", "UNSIGNED_LONG", "LONG_LONG", "UNSIGNED_LONG_LONG", "FLOAT", "DOUBLE",
                            "BOOL", "NONE_DATA_TYPE"};
  return n[(int)t];
}
const char *dtype_c_name(DType t) {
  switch (t) {
    case CHAR: return "signed char";
    case UNSIGNED_CHAR: return "unsigned char";
    case SHORT: return "short";
    case UNSIGNED_SHORT: return "unsigned short";
    case INT: return "int";
    case UNSIGNED_INT: return "unsigned int";
    case LONG: case LONG_LONG: return "long long";
    case UNSIGNED_LONG: case UNSIGNED_LONG_LONG: return "unsigned long long";
    case FLOAT: return "float";
    case DOUBLE: return "double";
    case BOOL: return "bool";
    default: return "void";
  }
}

// get_matrix_index_and_val_from_file (struct.cc:92-175): first non-blank line is
// "rows cols [nnz]", every further line "row col val", 1-based, rows
// non-decreasing.  Lines starting with white space are skipped, as upstream.
// Upstream takes whatever atol / stof make of a line (an index of 0 wraps to 2^64 - 1, an index beyond the header
// is kept); here every entry is checked against the header and a line that does not parse is an error, because
// the indices end up addressing x and y on the device.
CooInput read_coo_file(const std::string &path, DType val_dtype) {
  AS_CHECK(val_dtype == FLOAT || val_dtype == DOUBLE, "value type must be FLOAT or DOUBLE");
  std::ifstream in(path, std::ios::binary);
  AS_CHECK(in.is_open(), "cannot open file " + path);
  CooInput out;
  out.val_dtype = val_dtype;
  std::string line;
  bool first = true;
  uint64_t line_no = 0;
  while (std::getline(in, line)) {
    if (line.empty() || isspace((unsigned char)line[0])) continue;
    line_no++;
    const std::string where = path + ", entry line " + std::to_string(line_no);
    const char *p = line.c_str();
    char *e = nullptr;
    long a = strtol(p, &e, 10);
    AS_CHECK(e != p, "malformed line (no row index) in " + where);
    const char *q = e;
    long b = strtol(q, &e, 10);
    AS_CHECK(e != q, "malformed line (no column index) in " + where);
    if (first) {
      AS_CHECK(a > 0 && b > 0, "matrix sizes must be positive in " + path);
      out.row_index_max = (uint64_t)(a - 1);
      out.col_index_max = (uint64_t)(b - 1);
      first = false;
      continue;
    }
    AS_CHECK(a >= 1 && (uint64_t)a <= out.row_index_max + 1, "row index outside 1..rows in " + where);
    AS_CHECK(b >= 1 && (uint64_t)b <= out.col_index_max + 1, "column index outside 1..cols in " + where);
    uint64_t r = (uint64_t)(a - 1), c = (uint64_t)(b - 1);
    AS_CHECK(out.row.empty() || r >= out.row.back(), "row indices must be non-decreasing");
    out.row.push_back(r);
    out.col.push_back(c);
    // stof / stod semantics: the value is parsed at its own precision.
    q = e;
    const double v = val_dtype == DOUBLE ? strtod(q, &e) : (double)strtof(q, &e);
    AS_CHECK(e != q, "malformed line (no value) in " + where);
    out.val.push_back(v);
  }
  AS_CHECK(!first, "no header line in " + path);
  AS_CHECK(!out.row.empty(), "no entries in " + path);
  return out;
}

void write_coo_file(const std::string &path, uint64_t rows, uint64_t cols, const std::vector<uint64_t> &row,
                    const std::vector<uint64_t> &col, const ValVec &val, DType val_dtype) {
  FILE *f = fopen(path.c_str(), "w");
  AS_CHECK(f != nullptr, "cannot open file " + path);
  fprintf(f, "%lu %lu %lu\n", (unsigned long)rows, (unsigned long)cols, (unsigned long)row.size());
  for (size_t i = 0; i < row.size(); i++) {
    if (val_dtype == FLOAT)
      fprintf(f, "%lu %lu %.9g\n", (unsigned long)row[i] + 1, (unsigned long)col[i] + 1, (double)(float)val[i]);
    else
      fprintf(f, "%lu %lu %.17g\n", (unsigned long)row[i] + 1, (unsigned long)col[i] + 1, val[i]);
  }
  fclose(f);
}

// data_prepare.py:34-66 with the Matrix Market banner honoured (see matrix.hpp)
CooInput read_mtx_file(const std::string &path, DType val_dtype, bool keep_values) {
  AS_CHECK(val_dtype == FLOAT || val_dtype == DOUBLE, "value type must be FLOAT or DOUBLE");
  std::ifstream in(path, std::ios::binary);
  AS_CHECK(in.is_open(), "cannot open file " + path);
  CooInput out;
  out.val_dtype = val_dtype;
  std::string line;
  bool first = true, pattern = false, mirror = false, skew = false;
  uint64_t rows = 0, cols = 0;
  struct Entry { uint64_t r, c; double v; };
  std::vector<Entry> all;
  while (std::getline(in, line)) {
    if (line.empty()) continue;
    if (line[0] == '%') {
      if (line.compare(0, 14, "%%MatrixMarket") == 0) {
        std::string low(line);
        for (char &ch : low) ch = (char)tolower((unsigned char)ch);
        AS_CHECK(low.find("coordinate") != std::string::npos, "only coordinate Matrix Market files are supported");
        AS_CHECK(low.find("complex") == std::string::npos, "complex matrices are not supported");
        pattern = low.find("pattern") != std::string::npos;
        skew = low.find("skew-symmetric") != std::string::npos;
        mirror = skew || low.find("symmetric") != std::string::npos || low.find("hermitian") != std::string::npos;
      }
      continue;
    }
    const char *p = line.c_str();
    while (*p && isspace((unsigned char)*p)) p++;
    if (!*p) continue;
    char *e = nullptr;
    long a = strtol(p, &e, 10);
    AS_CHECK(e != p, "malformed line in " + path);
    const char *q = e;
    long b = strtol(q, &e, 10);
    AS_CHECK(e != q, "malformed line in " + path);
    if (first) {
      AS_CHECK(a > 0 && b > 0, "matrix sizes must be positive");
      rows = (uint64_t)a;
      cols = (uint64_t)b;
      long n = strtol(e, nullptr, 10);
      if (n > 0) all.reserve((size_t)n * (mirror ? 2 : 1));
      first = false;
      continue;
    }
    AS_CHECK(a >= 1 && (uint64_t)a <= rows && b >= 1 && (uint64_t)b <= cols, "entry outside the matrix in " + path);
    double v = 1.0;
    if (!pattern && keep_values) {
      q = e;
      v = val_dtype == DOUBLE ? strtod(q, &e) : (double)strtof(q, &e);
      AS_CHECK(e != q, "entry without a value in " + path);
    }
    all.push_back({(uint64_t)a - 1, (uint64_t)b - 1, v});
    if (mirror && a != b) all.push_back({(uint64_t)b - 1, (uint64_t)a - 1, skew && keep_values ? -v : v});
  }
  AS_CHECK(!first && !all.empty(), "file holds no element: " + path);
  std::stable_sort(all.begin(), all.end(), [](const Entry &x, const Entry &y) { return x.r != y.r ? x.r < y.r : x.c < y.c; });
  out.row_index_max = rows - 1;
  out.col_index_max = cols - 1;
  out.row.reserve(all.size());
  out.col.reserve(all.size());
  out.val.reserve(all.size());
  for (const Entry &en : all) {
    out.row.push_back(en.r);
    out.col.push_back(en.c);
    out.val.push_back(en.v);
  }
  return out;
}

namespace {
struct BinaryHeader {
  char magic[8];             // "ASXCOO1"
  uint64_t rows, cols, nnz;
  uint32_t val_dtype;        // DType ordinal: FLOAT or DOUBLE
  uint32_t index_bytes;      // 4 or 8
  uint64_t reserved[3];
};
static_assert(sizeof(BinaryHeader) == 64, "binary header must be 64 bytes");
}  // namespace

void write_coo_binary(const std::string &path, const CooInput &in) {
  AS_CHECK(in.row.size() == in.col.size() && in.row.size() == in.val.size() && !in.row.empty(), "malformed COO");
  FILE *f = fopen(path.c_str(), "wb");
  AS_CHECK(f != nullptr, "cannot open file " + path);
  BinaryHeader h = {};
  memcpy(h.magic, "ASXCOO1", 8);
  h.rows = in.row_index_max + 1;
  h.cols = in.col_index_max + 1;
  h.nnz = in.row.size();
  h.val_dtype = (uint32_t)in.val_dtype;
  h.index_bytes = (h.rows <= 0xffffffffull && h.cols <= 0xffffffffull) ? 4 : 8;
  bool ok = fwrite(&h, sizeof h, 1, f) == 1;
  auto put_index = [&](const std::vector<uint64_t> &v) {
    if (h.index_bytes == 8) return fwrite(v.data(), 8, v.size(), f) == v.size();
    std::vector<uint32_t> n(v.begin(), v.end());
    return fwrite(n.data(), 4, n.size(), f) == n.size();
  };
  ok = ok && put_index(in.row) && put_index(in.col);
  if (in.val_dtype == DOUBLE) {
    ok = ok && fwrite(in.val.data(), 8, in.val.size(), f) == in.val.size();
  } else {
    std::vector<float> n(in.val.begin(), in.val.end());
    ok = ok && fwrite(n.data(), 4, n.size(), f) == n.size();
  }
  ok = (fclose(f) == 0) && ok;
  AS_CHECK(ok, "short write to " + path);
}

CooInput read_coo_binary(const std::string &path) {
  FILE *f = fopen(path.c_str(), "rb");
  AS_CHECK(f != nullptr, "cannot open file " + path);
  struct Close { FILE *f; ~Close() { fclose(f); } } closer{f};
  BinaryHeader h;
  AS_CHECK(fread(&h, sizeof h, 1, f) == 1 && memcmp(h.magic, "ASXCOO1", 8) == 0, "not a binary COO file: " + path);
  AS_CHECK((h.val_dtype == (uint32_t)FLOAT || h.val_dtype == (uint32_t)DOUBLE) && (h.index_bytes == 4 || h.index_bytes == 8) &&
               h.rows > 0 && h.cols > 0 && h.nnz > 0, "corrupt header in " + path);
  // the arrays must be there in full before anything is allocated for them
  AS_CHECK(fseek(f, 0, SEEK_END) == 0, "cannot seek in " + path);
  const uint64_t want = sizeof h + h.nnz * (2ull * h.index_bytes + (h.val_dtype == (uint32_t)DOUBLE ? 8 : 4));
  AS_CHECK((uint64_t)ftell(f) == want, "binary COO file has the wrong length: " + path);
  AS_CHECK(fseek(f, sizeof h, SEEK_SET) == 0, "cannot seek in " + path);
  CooInput out;
  out.val_dtype = (DType)h.val_dtype;
  out.row_index_max = h.rows - 1;
  out.col_index_max = h.cols - 1;
  auto get_index = [&](std::vector<uint64_t> &v, uint64_t limit) {
    v.resize(h.nnz);
    if (h.index_bytes == 8) {
      AS_CHECK(fread(v.data(), 8, v.size(), f) == v.size(), "short read from " + path);
    } else {
      std::vector<uint32_t> n(h.nnz);
      AS_CHECK(fread(n.data(), 4, n.size(), f) == n.size(), "short read from " + path);
      std::copy(n.begin(), n.end(), v.begin());
    }
    for (uint64_t x : v) AS_CHECK(x < limit, "index outside the matrix in " + path);
  };
  get_index(out.row, h.rows);
  get_index(out.col, h.cols);
  out.val.resize(h.nnz);
  if (out.val_dtype == DOUBLE) {
    AS_CHECK(fread(out.val.data(), 8, out.val.size(), f) == out.val.size(), "short read from " + path);
  } else {
    std::vector<float> n(h.nnz);
    AS_CHECK(fread(n.data(), 4, n.size(), f) == n.size(), "short read from " + path);
    std::copy(n.begin(), n.end(), out.val.begin());
  }
  return out;
}

// check_begin_memory_cache_input_file (exe_graph.cc:3850-3914)
bool check_coo_sorted(const CooInput &in) {
  AS_CHECK(in.row.size() == in.col.size() && in.row.size() == in.val.size() && !in.row.empty(), "malformed COO");
  for (size_t i = 1; i < in.row.size(); i++) {
    if (in.row[i] < in.row[i - 1]) return false;
    if (in.row[i] == in.row[i - 1] && in.col[i] < in.col[i - 1]) return false;
  }
  return true;
}

// has_empty_line_in_begin_memory_cache_input_file (exe_graph.cc:3916-3946).
// Rows are sorted, so distinct rows are counted in one pass instead of a set.
bool coo_has_empty_row(const CooInput &in) {
  AS_CHECK(!in.row.empty(), "malformed COO");
  uint64_t distinct = 1;
  bool sorted = true;
  for (size_t i = 1; i < in.row.size(); i++) {
    if (in.row[i] < in.row[i - 1]) { sorted = false; break; }
    if (in.row[i] != in.row[i - 1]) distinct++;
  }
  if (!sorted) {
    std::vector<uint64_t> r(in.row);
    std::sort(r.begin(), r.end());
    distinct = std::unique(r.begin(), r.end()) - r.begin();
  }
  return distinct != in.row_index_max + 1;
}

// init_sparse_struct_by_coo_vector (struct.cc:296-390)
std::unique_ptr<Matrix> matrix_from_coo(const CooInput &in, unsigned wave) {
  AS_CHECK(in.val_dtype == FLOAT || in.val_dtype == DOUBLE, "value type must be FLOAT or DOUBLE");
  AS_CHECK(!in.row.empty() && in.row.size() == in.col.size() && in.row.size() == in.val.size(), "malformed COO");
  AS_CHECK(wave == 32 || wave == 64, "wave must be 32 or 64");
  // every entry path ends here: no index may point outside x or y
  for (size_t i = 0; i < in.row.size(); i++)
    AS_CHECK(in.row[i] <= in.row_index_max && in.col[i] <= in.col_index_max, "entry " + std::to_string(i) + " lies outside the matrix");
  auto m = std::make_unique<Matrix>();
  m->rows = m->y_rows = in.row_index_max + 1;
  m->cols = in.col_index_max + 1;
  m->nnz = m->origin_nnz = in.row.size();
  m->coo_row = in.row;
  m->coo_col = in.col;
  m->coo_val = in.val;
  m->val_dtype = in.val_dtype;
  m->wave = wave;
  if (in.val_dtype == FLOAT)
    for (double &v : m->coo_val) v = (double)(float)v;
  return m;
}

std::unique_ptr<CompressedBlock> CompressedBlock::clone() const {
  auto c = std::make_unique<CompressedBlock>();
  c->share_row_with_other_block = share_row_with_other_block;
  c->share_row_with_other_warp = share_row_with_other_warp;
  c->share_row_with_other_thread = share_row_with_other_thread;
  c->val_dtype = val_dtype;
  c->col_slice = col_slice;
  c->row_group = row_group;
  c->is_sorted = is_sorted;
  c->y_write_index = y_write_index;
  // keep aliasing (nnz-div: slots 5/6 alias slot 1, padded values alias val)
  std::vector<std::pair<const Index *, IndexPtr>> seen;
  for (auto &ip : read_index) {
    IndexPtr n;
    for (auto &s : seen)
      if (s.first == ip.get()) n = s.second;
    if (!n) {
      n = std::make_shared<Index>(*ip);
      seen.emplace_back(ip.get(), n);
    }
    c->read_index.push_back(n);
  }
  if (val) c->val = std::make_shared<ValVec>(*val);
  auto dup = [&](const ValPtr &p) -> ValPtr {
    if (!p) return nullptr;
    if (p == val) return c->val;
    return std::make_shared<ValVec>(*p);
  };
  c->padding_val = dup(padding_val);
  c->staggered_val = (staggered_val && staggered_val == padding_val) ? c->padding_val : dup(staggered_val);
  return c;
}

std::unique_ptr<Matrix> Matrix::clone() const {
  auto m = std::make_unique<Matrix>();
  m->rows = rows; m->cols = cols; m->nnz = nnz; m->origin_nnz = origin_nnz;
  m->y_rows = y_rows; m->rows_compacted = rows_compacted;
  m->is_compressed = is_compressed; m->is_blocked = is_blocked; m->is_sorted = is_sorted;
  m->sorted_row_index = sorted_row_index;
  m->coo_row = coo_row; m->coo_col = coo_col; m->coo_val = coo_val;
  m->val_dtype = val_dtype; m->wave = wave; m->val_copy_from_zero_quirk = val_copy_from_zero_quirk;
  for (auto &it : items) {
    DenseItem d;
    d.min_row = it.min_row; d.max_row = it.max_row; d.min_col = it.min_col; d.max_col = it.max_col;
    d.begin_coo = it.begin_coo; d.end_coo = it.end_coo; d.is_col_blocked = it.is_col_blocked;
    if (it.cb) d.cb = it.cb->clone();
    m->items.push_back(std::move(d));
  }
  return m;
}

std::unique_ptr<Matrix> Matrix::clone_for_sub(uint64_t sub) const {
  AS_CHECK(sub < items.size() && items[sub].cb, "sub-matrix is not compressed");
  auto m = std::make_unique<Matrix>();
  m->rows = rows; m->cols = cols; m->nnz = nnz; m->origin_nnz = origin_nnz;
  m->y_rows = y_rows; m->rows_compacted = rows_compacted;
  m->is_compressed = is_compressed; m->is_blocked = is_blocked; m->is_sorted = is_sorted;
  m->sorted_row_index = sorted_row_index;
  m->val_dtype = val_dtype; m->wave = wave; m->val_copy_from_zero_quirk = val_copy_from_zero_quirk;
  for (size_t i = 0; i < items.size(); i++) {
    const DenseItem &it = items[i];
    DenseItem d;
    d.min_row = it.min_row; d.max_row = it.max_row; d.min_col = it.min_col; d.max_col = it.max_col;
    d.begin_coo = it.begin_coo; d.end_coo = it.end_coo; d.is_col_blocked = it.is_col_blocked;
    if (i == sub) d.cb = it.cb->clone();
    m->items.push_back(std::move(d));
  }
  return m;
}

}  // namespace asx
