// extern "C" surface: code builder, kernel templates, execution.
#include <cstring>

#include "capi_internal.hpp"
#include "code_builder.hpp"
#include "hip_layer.h"
#include "search.hpp"

struct as_builder {
  std::unique_ptr<asx::Matrix> owned_matrix;  // set when the builder was rebuilt from a search result
  std::unique_ptr<asx::Builder> b;            // destroyed before owned_matrix
  std::string text;                           // backing store of returned strings
};

struct as_search_result {
  asx::SearchResult r;
  std::string report;
};

static asx::Template &tpl_of(as_builder *b, int64_t sub) {
  AS_CHECK(b && b->b, "null builder");
  AS_CHECK(sub >= 0 && (uint64_t)sub < b->b->subs.size() && b->b->subs[sub].tpl, "sub-matrix has no template");
  return *b->b->subs[sub].tpl;
}

extern "C" {

as_builder *as_builder_create(const as_matrix *m) {
  AS_API_BEGIN
  AS_CHECK(m && m->m, "null matrix");
  auto *h = new as_builder();
  h->b = asx::init_code_builder(*m->m);
  return h;
  AS_API_END(nullptr)
}

void as_builder_free(as_builder *b) { delete b; }

int as_template_is_supported(const as_matrix *m, int64_t sub, int template_type) {
  AS_API_BEGIN
  AS_CHECK(m && m->m && sub >= 0, "bad argument");
  return asx::is_supported_by_template((asx::TemplateType)template_type, *m->m, (uint64_t)sub) ? 1 : 0;
  AS_API_END(-1)
}

int as_builder_set_template(as_builder *b, int64_t sub, int template_type) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && sub >= 0, "bad argument");
  asx::add_template_to_builder(*b->b, (uint64_t)sub, (asx::TemplateType)template_type);
  return 0;
  AS_API_END(-1)
}

int as_builder_compress(as_builder *b, int64_t sub) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && sub >= 0, "bad argument");
  return asx::compress_template_in_builder(*b->b, (uint64_t)sub) ? 1 : 0;
  AS_API_END(-1)
}

int as_builder_set_launch(as_builder *b, int64_t sub, long tblock_num, long thread_num_in_block,
                          long thread_num_of_row_reduce, long vec_width) {
  AS_API_BEGIN
  asx::Template &t = tpl_of(b, sub);
  if (vec_width > 0) {
    AS_CHECK(vec_width == 1 || vec_width == 2 || vec_width == 4, "vec_width must be 1, 2 or 4");
    t.vec_width = (unsigned)vec_width;
    if (thread_num_in_block <= 0) t.thread_num_in_block = 0;  // re-derive the default block size
  }
  if (thread_num_in_block > 0) {
    AS_CHECK(thread_num_in_block % 64 == 0 && thread_num_in_block <= 1024, "threads per block: multiple of 64, <= 1024");
    t.thread_num_in_block = (uint64_t)thread_num_in_block;
  }
  // the grid that covers the format follows from block size and vector width
  asx::set_default_launch(t);
  if (tblock_num > 0) t.tblock_num = (uint64_t)tblock_num;
  if (thread_num_of_row_reduce > 0) t.thread_num_of_row_reduce = (uint64_t)thread_num_of_row_reduce;
  asx::invalidate_module(*b->b);  // arrays stay resident; only the module is rebuilt
  return 0;
  AS_API_END(-1)
}

int as_builder_set_relative_columns(as_builder *b, int64_t sub) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && sub >= 0, "bad argument");
  return asx::set_relative_columns(*b->b, (uint64_t)sub) ? 1 : 0;
  AS_API_END(-1)
}

int as_builder_set_diagonal_columns(as_builder *b, int64_t sub) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && sub >= 0, "bad argument");
  return asx::set_diagonal_columns(*b->b, (uint64_t)sub) ? 1 : 0;
  AS_API_END(-1)
}

int as_builder_set_row_ownership(as_builder *b, int64_t sub) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && sub >= 0, "bad argument");
  return asx::set_row_ownership(*b->b, (uint64_t)sub) ? 1 : 0;
  AS_API_END(-1)
}

int as_builder_set_row_blocks(as_builder *b, int64_t sub, int rows_per_block) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && sub >= 0 && rows_per_block >= 2 && rows_per_block <= 4, "bad argument");
  return asx::set_row_blocks(*b->b, (uint64_t)sub, (uint64_t)rows_per_block) ? 1 : 0;
  AS_API_END(-1)
}

int as_builder_set_column_runs(as_builder *b, int64_t sub) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && sub >= 0, "bad argument");
  return asx::set_column_runs(*b->b, (uint64_t)sub) ? 1 : 0;
  AS_API_END(-1)
}

int as_builder_get_launch(as_builder *b, int64_t sub, long out[4]) {
  AS_API_BEGIN
  asx::Template &t = tpl_of(b, sub);
  out[0] = (long)t.tblock_num; out[1] = (long)t.thread_num_in_block; out[2] = (long)t.thread_num_of_row_reduce;
  out[3] = (long)t.vec_width;
  return 0;
  AS_API_END(-1)
}

// arrays of a template by name; "val_arr" through as_template_get_f64, "col_index_arr" and metadata here
int64_t as_template_get_u64(as_builder *b, int64_t sub, const char *name, uint64_t *out, uint64_t cap, int *dtype,
                            int *compress_type) {
  AS_API_BEGIN
  asx::Template &t = tpl_of(b, sub);
  AS_CHECK(name, "null name");
  const asx::IArr *a = nullptr;
  int ct = asx::NONE_COMPRESS;
  if (!strcmp(name, "col_index_arr")) a = &t.col_index_arr;
  else if (asx::TArr *p = t.find(name)) { a = &p->a; ct = p->c.type; }
  if (!a) return -1;
  if (dtype) *dtype = (int)a->dt;
  if (compress_type) *compress_type = ct;
  if (out) memcpy(out, a->v.data(), sizeof(uint64_t) * std::min<uint64_t>(cap, a->size()));
  return (int64_t)a->size();
  AS_API_END(-2)
}

int64_t as_template_get_f64(as_builder *b, int64_t sub, double *out, uint64_t cap) {
  AS_API_BEGIN
  asx::Template &t = tpl_of(b, sub);
  if (out) memcpy(out, t.val_arr.data(), sizeof(double) * std::min<uint64_t>(cap, t.val_arr.size()));
  return (int64_t)t.val_arr.size();
  AS_API_END(-2)
}

// "name=value" lines: scalars, flags, array names with dtype and compression
const char *as_template_describe(as_builder *b, int64_t sub) {
  AS_API_BEGIN
  asx::Template &t = tpl_of(b, sub);
  std::string s = std::string("template=") + asx::convert_template_type_to_string(t.type) + "\n";
  s += "kernal_first_row_index=" + std::to_string(t.kernal_first_row_index) + "\n";
  s += "kernal_first_col_index=" + std::to_string(t.kernal_first_col_index) + "\n";
  s += "is_atom_add=" + std::to_string((int)t.is_atom_add) + "\n";
  s += "global_sort_index=" + std::to_string((int)t.global_sort_index) + "\n";
  s += "local_sort_index=" + std::to_string((int)t.local_sort_index) + "\n";
  for (auto &kv : t.scalar) s += kv.first + "=" + std::to_string(kv.second) + "\n";
  for (auto &a : t.arrays)
    s += "array:" + a.name + "=" + asx::dtype_name(a.a.dt) + "," + std::to_string(a.a.size()) + "," +
         asx::compress_type_name(a.c.type) + "\n";
  s += "array:col_index_arr=" + std::string(asx::dtype_name(t.col_index_arr.dt)) + "," + std::to_string(t.col_index_arr.size()) + ",NONE_COMPRESS\n";
  s += "array:val_arr=" + std::string(asx::dtype_name(t.val_dtype)) + "," + std::to_string(t.val_arr.size()) + ",NONE_COMPRESS\n";
  b->text = s;
  return b->text.c_str();
  AS_API_END(nullptr)
}

const char *as_builder_kernel_source(as_builder *b) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  b->text = asx::build_module_source(*b->b);
  return b->text.c_str();
  AS_API_END(nullptr)
}

int as_builder_compile(as_builder *b) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  asx::compile_builder(*b->b);
  return 0;
  AS_API_END(-1)
}

int as_builder_upload(as_builder *b, int device) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  asx::load_and_upload(*b->b, device);
  return 0;
  AS_API_END(-1)
}

int as_builder_spmv(as_builder *b, const void *x_host, void *y_host) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && x_host && y_host, "null argument");
  asx::spmv_host(*b->b, x_host, y_host);
  return 0;
  AS_API_END(-1)
}

int as_builder_spmv_device(as_builder *b, const void *x_dev, void *y_dev) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && x_dev && y_dev, "null argument");
  asx::launch_spmv(*b->b, x_dev, y_dev);
  if (as_hip_stream_sync(b->b->main_stream) != 0) throw asx::Error(as_hip_last_error());
  return 0;
  AS_API_END(-1)
}

int as_builder_spmv_device_no_alloc(as_builder *b, const void *x_dev, void *y_dev) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && x_dev && y_dev, "null argument");
  asx::launch_spmv_no_alloc(*b->b, x_dev, y_dev);
  if (as_hip_stream_sync(b->b->main_stream) != 0) throw asx::Error(as_hip_last_error());
  return 0;
  AS_API_END(-1)
}

int as_builder_spmv_device_async(as_builder *b, const void *x_dev, void *y_dev, void *stream) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && x_dev && y_dev, "null argument");
  asx::launch_spmv(*b->b, x_dev, y_dev, stream);
  return 0;
  AS_API_END(-1)
}

int as_builder_spmv_device_no_alloc_async(as_builder *b, const void *x_dev, void *y_dev, void *stream) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && x_dev && y_dev, "null argument");
  asx::launch_spmv_no_alloc(*b->b, x_dev, y_dev, stream);
  return 0;
  AS_API_END(-1)
}

void *as_builder_stream(as_builder *b) { return b && b->b ? b->b->main_stream : nullptr; }

int64_t as_builder_static_scratch_need(as_builder *b) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  return (int64_t)asx::static_scratch_need(*b->b);
  AS_API_END(-1)
}

int as_builder_clears_y(as_builder *b) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  return asx::y_needs_clear(*b->b) ? 1 : 0;
  AS_API_END(-1)
}

int as_builder_set_x(as_builder *b, const void *x_host) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && x_host && b->b->device_ready, "builder is not on the device");
  if (as_hip_h2d(b->b->x.ptr, x_host, b->b->x.bytes) != 0) throw asx::Error(as_hip_last_error());
  return 0;
  AS_API_END(-1)
}

// Back-to-back launches of the kernels of ONE sub-matrix (events on the launch stream): the per-kernel
// duration and bytes that a roofline figure of a multi-strip graph is quoted on.  format_bytes = padded
// col + val + passed metadata (+ scratch traffic); rows = rows of the strip; atom = y accumulated atomically.
int as_builder_time_sub_matrix(as_builder *b, int64_t sub, uint64_t reps, float *time_ms, uint64_t *format_bytes,
                               uint64_t *rows, int *atom) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && time_ms && reps > 0, "bad argument");
  asx::Builder &bd = *b->b;
  AS_CHECK(sub >= 0 && (uint64_t)sub < bd.subs.size() && bd.subs[sub].tpl, "sub-matrix has no template");
  struct Reset { asx::Builder &bd; ~Reset() { bd.only_sub = -1; } } reset{bd};
  bd.only_sub = sub;
  float gf = 0;
  asx::time_spmv(bd, reps, false, *time_ms, gf);
  const asx::Template &t = *bd.subs[sub].tpl;
  if (format_bytes) *format_bytes = asx::template_format_bytes(t);
  if (rows) *rows = bd.matrix ? bd.matrix->items[sub].max_row - bd.matrix->items[sub].min_row + 1 : 0;
  if (atom) *atom = t.is_atom_add ? 1 : 0;
  return 0;
  AS_API_END(-1)
}

int as_builder_time_sub_matrix_pass(as_builder *b, int64_t sub, int pass, uint64_t reps, float *time_ms) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && time_ms && reps > 0 && (pass == 1 || pass == 2), "bad argument");
  asx::Builder &bd = *b->b;
  AS_CHECK(sub >= 0 && (uint64_t)sub < bd.subs.size() && bd.subs[sub].tpl, "sub-matrix has no template");
  AS_CHECK(bd.subs[sub].tpl->finish_tblock_num, "the template of this sub-matrix has one kernel only");
  struct Reset { asx::Builder &bd; ~Reset() { bd.only_sub = -1; bd.only_pass = 0; } } reset{bd};
  bd.only_sub = sub;
  bd.only_pass = pass;
  float gf = 0;
  asx::time_spmv(bd, reps, false, *time_ms, gf);
  // a first kernel that adds into a scratch vector its finish kernel leaves cleared: cleared here instead
  if (pass == 1 && bd.subs[sub].tpl->scratch_starts_zero) asx::clear_scratch(bd, (uint64_t)sub);
  return 0;
  AS_API_END(-1)
}

int as_kernel_cache_stats(uint64_t *entries, uint64_t *hits) {
  AS_API_BEGIN
  AS_CHECK(entries && hits, "null argument");
  asx::code_cache_stats(*entries, *hits);
  return 0;
  AS_API_END(-1)
}

int as_builder_set_serial_launch(as_builder *b, int serial) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  if (b->b->serial_launch != (serial != 0)) asx::invalidate_module(*b->b);  // which finish kernels are carried changes
  b->b->serial_launch = serial != 0;
  return 0;
  AS_API_END(-1)
}

int as_builder_set_finish_carry(as_builder *b, int on) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  if (b->b->carry_finish != (on != 0)) asx::invalidate_module(*b->b);
  b->b->carry_finish = on != 0;
  return 0;
  AS_API_END(-1)
}

int as_builder_set_fuse_launches(as_builder *b, int on) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  if (b->b->fuse_launches != (on != 0)) asx::invalidate_module(*b->b);
  b->b->fuse_launches = on != 0;
  return 0;
  AS_API_END(-1)
}

int as_builder_launch_is_fused(as_builder *b, uint64_t sub) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  AS_CHECK(sub < b->b->subs.size() && b->b->subs[sub].tpl, "sub-matrix has no template");
  asx::assign_finish_carriers(*b->b, sub);
  for (auto &k : b->b->subs)
    if (k.tpl && k.tpl->fused_trips == b->b->subs[sub].tpl.get()) return 1;
  return 0;
  AS_API_END(-1)
}

int as_builder_finish_carrier(as_builder *b, uint64_t sub, int64_t *carrier) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && carrier, "null argument");
  AS_CHECK(sub < b->b->subs.size() && b->b->subs[sub].tpl, "sub-matrix has no template");
  *carrier = asx::assign_finish_carriers(*b->b, sub);
  return 0;
  AS_API_END(-1)
}

int as_builder_time(as_builder *b, uint64_t reps, int sync_each_launch, float *time_ms, float *gflops) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && time_ms && gflops, "null argument");
  asx::time_spmv(*b->b, reps, sync_each_launch != 0, *time_ms, *gflops);
  return 0;
  AS_API_END(-1)
}

int64_t as_builder_scratch_bytes(as_builder *b, int64_t sub) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  uint64_t bytes = 0;
  for (size_t s = 0; s < b->b->subs.size(); s++)
    if (b->b->subs[s].tpl && (sub < 0 || (int64_t)s == sub)) bytes += b->b->subs[s].tpl->scratch_bytes;
  return (int64_t)bytes;
  AS_API_END(-1)
}

int64_t as_builder_algorithmic_bytes(as_builder *b) {
  AS_API_BEGIN
  AS_CHECK(b && b->b, "null builder");
  return (int64_t)asx::builder_algorithmic_bytes(*b->b);
  AS_API_END(-1)
}

}  // extern "C"

// Self-test of the wave-level reduction helpers that every generated kernel
// uses: runs as_group_sum<lanes> (DPP) and as_group_sum_shfl<lanes> on one
// 64-lane wavefront holding `in[lane]` and returns both per-lane results.
extern "C" int as_selftest_group_sum(int device, int lanes, int is_double, const double *in, double *dpp_out,
                                     double *shfl_out) {
  AS_API_BEGIN
  AS_CHECK(in && dpp_out && shfl_out, "null argument");
  AS_CHECK(lanes == 1 || lanes == 2 || lanes == 4 || lanes == 8 || lanes == 16 || lanes == 32 || lanes == 64, "bad lanes");
  std::string T = is_double ? "double" : "float", L = std::to_string(lanes);
  std::string src = asx::kernel_module_preamble() +
                    "extern \"C\" __global__ void selftest(const double *in, double *a, double *b)\n{\n  " + T +
                    " v = (" + T + ")in[threadIdx.x];\n  a[threadIdx.x] = (double)as_group_sum<" + L +
                    ">(v);\n  b[threadIdx.x] = (double)as_group_sum_shfl<" + L + ">(v);\n}\n";
  void *code = nullptr, *mod = nullptr, *fn = nullptr, *din = nullptr, *da = nullptr, *db = nullptr;
  uint64_t n = 0;
  auto H = [](int r) { if (r != 0) throw asx::Error(as_hip_last_error()); };
  H(as_hip_compile(src.c_str(), "gfx950", nullptr, 0, &code, &n, nullptr));
  H(as_hip_init(device));
  H(as_hip_module_load(code, &mod));
  as_hip_free_host(code);
  H(as_hip_get_kernel(mod, "selftest", &fn));
  H(as_hip_alloc(&din, 64 * 8)); H(as_hip_alloc(&da, 64 * 8)); H(as_hip_alloc(&db, 64 * 8));
  H(as_hip_h2d(din, in, 64 * 8));
  void *args[] = {&din, &da, &db};
  H(as_hip_launch(fn, 1, 64, 0, nullptr, args));
  H(as_hip_device_sync());
  H(as_hip_d2h(dpp_out, da, 64 * 8));
  H(as_hip_d2h(shfl_out, db, 64 * 8));
  as_hip_free(din); as_hip_free(da); as_hip_free(db);
  as_hip_module_unload(mod);
  return 0;
  AS_API_END(-1)
}

// Self-test of the segmented sum the tile kernel reduces row runs with: one 64-lane wavefront holds
// (key[lane], in[lane]), keys sorted along the lanes; returns as_wave_segmented_sum per lane and
// as_is_segment_tail per lane (1.0 / 0.0).
extern "C" int as_selftest_segmented_sum(int device, int is_double, const unsigned *key, const double *in, double *sum_out,
                                         double *tail_out) {
  AS_API_BEGIN
  AS_CHECK(key && in && sum_out && tail_out, "null argument");
  for (int i = 0; i < 64; i++) AS_CHECK(key[i] != 0xffffffffu && (i == 0 || key[i] >= key[i - 1]), "keys must be sorted and not 0xffffffff");
  std::string T = is_double ? "double" : "float";
  std::string src = asx::kernel_module_preamble() +
                    "extern \"C\" __global__ void selftest(const unsigned int *key, const double *in, double *a, double *b)\n{\n  " + T +
                    " v = (" + T + ")in[threadIdx.x];\n  const unsigned int k = key[threadIdx.x];\n"
                    "  a[threadIdx.x] = (double)as_wave_segmented_sum(k, v);\n  b[threadIdx.x] = as_is_segment_tail(k) ? 1.0 : 0.0;\n}\n";
  void *code = nullptr, *mod = nullptr, *fn = nullptr, *dk = nullptr, *din = nullptr, *da = nullptr, *db = nullptr;
  uint64_t n = 0;
  auto H = [](int r) { if (r != 0) throw asx::Error(as_hip_last_error()); };
  H(as_hip_compile(src.c_str(), "gfx950", nullptr, 0, &code, &n, nullptr));
  H(as_hip_init(device));
  H(as_hip_module_load(code, &mod));
  as_hip_free_host(code);
  H(as_hip_get_kernel(mod, "selftest", &fn));
  H(as_hip_alloc(&dk, 64 * 4)); H(as_hip_alloc(&din, 64 * 8)); H(as_hip_alloc(&da, 64 * 8)); H(as_hip_alloc(&db, 64 * 8));
  H(as_hip_h2d(dk, key, 64 * 4));
  H(as_hip_h2d(din, in, 64 * 8));
  void *args[] = {&dk, &din, &da, &db};
  H(as_hip_launch(fn, 1, 64, 0, nullptr, args));
  H(as_hip_device_sync());
  H(as_hip_d2h(sum_out, da, 64 * 8));
  H(as_hip_d2h(tail_out, db, 64 * 8));
  as_hip_free(dk); as_hip_free(din); as_hip_free(da); as_hip_free(db);
  as_hip_module_unload(mod);
  return 0;
  AS_API_END(-1)
}

// arr_optimization.cc: try one compressor on an array.  type = enum arr_compress_type ordinal
// (1 LINEAR, 2 CONSTANT, 3 BRANCH, 4 CYCLE_LINEAR (param = cycle), 5 CYCLE_INCREASE).
// Returns 1 and fills out = {coefficient, intercept, constant, cycle, branches} when the array
// follows the pattern, 0 when it does not; eval[i] (optional, n entries) receives the closed form
// evaluated at i; code (optional) the emitted read expression "v = <expr of i>".
extern "C" int as_compress_array(const uint64_t *values, uint64_t n, int type, uint64_t param, uint64_t out[5],
                                 uint64_t *eval, char *code, uint64_t code_cap) {
  AS_API_BEGIN
  AS_CHECK(values && n > 0 && out, "null argument");
  asx::IArr a;
  a.assign(std::vector<uint64_t>(values, values + n), asx::UNSIGNED_LONG);
  asx::Compressor c;
  bool ok = false;
  switch ((asx::ArrCompressType)type) {
    case asx::LINEAR_COMPRESS: ok = asx::init_linear_compressor(a, c, true); break;
    case asx::CONSTANT_COMPRESS: ok = asx::init_constant_compressor(a, c, true); break;
    case asx::BRANCH_COMPRESS: ok = n > 2 && asx::init_branch_compressor(a, c, param ? param : 5); break;
    case asx::CYCLE_LINEAR_COMPRESS: ok = asx::init_cycle_linear_compressor(a, param, c, true); break;
    case asx::CYCLE_INCREASE_COMPRESS: ok = asx::init_cycle_increase_compressor(a, c, true); break;
    default: throw asx::Error("unknown compress type");
  }
  if (!ok) return 0;
  out[0] = c.coefficient; out[1] = c.intercept; out[2] = c.constant; out[3] = c.cycle; out[4] = c.low.size();
  if (eval)
    for (uint64_t i = 0; i < n; i++) eval[i] = c.eval(i);
  if (code && code_cap) {
    std::string s = asx::code_of_arr_read(c, "v", "i");
    strncpy(code, s.c_str(), code_cap - 1);
    code[code_cap - 1] = 0;
  }
  return 1;
  AS_API_END(-1)
}


// ---- executor.hpp:12-24 ------------------------------------------------------------------------
extern "C" {

static asx::CooInput coo_of(const as_matrix *m) {
  AS_CHECK(m && m->m, "null matrix");
  AS_CHECK(!m->m->is_compressed && !m->m->is_sorted && m->m->items.empty(), "need the matrix as read from the input (no operator applied)");
  asx::CooInput in;
  in.row = m->m->coo_row; in.col = m->m->coo_col; in.val = m->m->coo_val;
  in.row_index_max = m->m->rows - 1; in.col_index_max = m->m->cols - 1; in.val_dtype = m->m->val_dtype;
  return in;
}

int as_part_execute_code_builder(as_builder *b, const int64_t *sub_matrix_ids, uint64_t n_ids, uint64_t repeat,
                                 float *time_ms, float *gflops) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && time_ms && gflops, "bad argument");
  asx::Builder &bd = *b->b;
  AS_CHECK(bd.device_ready, "builder is not on the device");
  // run only the listed sub-matrices: the templates of the others are parked for the call
  std::vector<std::unique_ptr<asx::Template>> parked(bd.subs.size());
  std::vector<bool> keep(bd.subs.size(), n_ids == 0);
  for (uint64_t i = 0; i < n_ids; i++) {
    AS_CHECK(sub_matrix_ids && sub_matrix_ids[i] >= 0 && (uint64_t)sub_matrix_ids[i] < bd.subs.size(), "sub-matrix id out of range");
    keep[sub_matrix_ids[i]] = true;
  }
  bool changed = false;
  for (size_t s = 0; s < bd.subs.size(); s++)
    if (!keep[s] && bd.subs[s].tpl) { parked[s] = std::move(bd.subs[s].tpl); changed = true; }
  struct Restore {
    asx::Builder &bd; std::vector<std::unique_ptr<asx::Template>> &parked; bool changed;
    ~Restore() {
      for (size_t s = 0; s < parked.size(); s++)
        if (parked[s]) bd.subs[s].tpl = std::move(parked[s]);
      if (changed) asx::invalidate_module(bd);
    }
  } restore{bd, parked, changed};
  if (changed) asx::invalidate_module(bd);
  if (repeat == 0) {
    // the reference's own count (executor.cc:247-255): 185.2 G padded elements in all, at least two launches
    uint64_t total_nnz = 0;
    for (auto &k : bd.subs)
      if (k.tpl) total_nnz += k.tpl->padding_arr_size;
    AS_CHECK(total_nnz > 0, "no sub-matrix has a template");
    repeat = std::max<uint64_t>(2, 185200000000ull / total_nnz);
  }
  asx::time_spmv(bd, repeat, true, *time_ms, *gflops);  // kernel; synchronize -- as the upstream timing loop
  return 0;
  AS_API_END(-1)
}

int as_execute_code_builder(as_builder *b, double seconds, uint64_t *repeat_out, float *time_ms, float *gflops) {
  AS_API_BEGIN
  AS_CHECK(b && b->b && time_ms && gflops && seconds > 0, "bad argument");
  float ms = 0, gf = 0;
  asx::time_spmv(*b->b, 3, false, ms, gf);
  asx::time_spmv(*b->b, 10, false, ms, gf);
  uint64_t reps = (uint64_t)std::max(2.0, seconds * 1e3 / std::max(1e-4, (double)ms / 10.0));
  asx::time_spmv(*b->b, reps, false, *time_ms, *gflops);
  if (repeat_out) *repeat_out = reps;
  return 0;
  AS_API_END(-1)
}

as_search_result *as_find_best_graph(const as_matrix *input, const as_search_options *o) {
  AS_API_BEGIN
  asx::CooInput in = coo_of(input);
  asx::SearchOptions opt;
  if (o) {
    if (o->total_time_s > 0) opt.total_time_s = o->total_time_s;
    if (o->struggle_step_num > 0) opt.struggle_step_num = o->struggle_step_num;
    if (o->padding_rate_up_bound > 0) opt.padding_rate_up_bound = o->padding_rate_up_bound;
    opt.device = o->device;
    if (o->timed_region_ms > 0) opt.timed_region_ms = o->timed_region_ms;
    if (o->checkpoint_dir) opt.checkpoint_dir = o->checkpoint_dir;
    opt.verbose = o->verbose != 0;
    opt.only_dense_strategy = o->only_dense_strategy;
    opt.remove_empty_rows = o->remove_empty_rows != 0;
    opt.general_templates = o->general_templates != 0;
    opt.verify_candidates = o->skip_verification == 0;
  }
  opt.wave = input->m->wave;
  auto *r = new as_search_result();
  try {
    r->r = asx::find_best_graph_of_white_list_strategy(in, opt);
  } catch (...) {
    delete r;
    throw;
  }
  r->report = asx::convert_graph_to_string(r->r.best);
  return r;
  AS_API_END(nullptr)
}

void as_search_free(as_search_result *r) { delete r; }
const char *as_search_report(const as_search_result *r) { return r ? r->report.c_str() : ""; }
const char *as_search_log(const as_search_result *r) { return r ? r->r.log.c_str() : ""; }

int64_t as_search_best_graph(const as_search_result *r, long *desc, uint64_t cap) {
  AS_API_BEGIN
  AS_CHECK(r, "null argument");
  std::vector<long> d;
  auto nodes = [&](const std::vector<asx::StrategyNode> &v) {
    d.push_back((long)v.size());
    for (const asx::StrategyNode &n : v) {
      d.push_back((long)n.strategy);
      if (n.strategy == asx::DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY) {
        d.push_back((long)n.in_nnz); d.push_back((long)n.in_val_dtype);
        d.push_back((long)n.in_col_index_max); d.push_back((long)n.in_row_index_max);
      } else {
        for (int i = 0; i < 4; i++) d.push_back(n.p[i]);
      }
    }
  };
  nodes(r->r.best.dense);
  d.push_back((long)r->r.best.subs.size());
  for (const asx::SubGraph &sub : r->r.best.subs) {
    nodes(sub.nodes);
    d.push_back((long)sub.tpl.type); d.push_back(sub.tpl.tblock_num);
    d.push_back(sub.tpl.thread_num_in_block); d.push_back(sub.tpl.thread_num_of_row_reduce);
  }
  if (desc)
    for (size_t i = 0; i < d.size() && i < cap; i++) desc[i] = d[i];
  return (int64_t)d.size();
  AS_API_END(-1)
}

int as_search_stats(const as_search_result *r, double out[8]) {
  AS_API_BEGIN
  AS_CHECK(r && out, "null argument");
  out[0] = r->r.best.gflops; out[1] = r->r.best.time_ms; out[2] = (double)r->r.candidates;
  out[3] = (double)r->r.failed_candidates; out[4] = r->r.seconds; out[5] = r->r.seconds_to_best;
  out[6] = (double)r->r.best.subs.size();
  out[7] = r->r.best.dense_strategy_name == "strategy1" ? 1 : r->r.best.dense_strategy_name == "strategy2" ? 2 : 3;
  return 0;
  AS_API_END(-1)
}

as_builder *as_search_build_best(const as_search_result *r, const as_matrix *input) {
  AS_API_BEGIN
  AS_CHECK(r, "null search result");
  asx::CooInput in = coo_of(input);
  asx::BuiltGraph g = asx::build_from_graph(in, r->r.best, input->m->wave);
  auto *h = new as_builder();
  h->owned_matrix = std::move(g.matrix);
  h->b = std::move(g.builder);
  return h;
  AS_API_END(nullptr)
}

}  // extern "C"

// Plain device-to-device copy kernel of a known size (`bytes` read + `bytes` written per launch,
// `reps` launches).  Used to calibrate the FETCH_SIZE / WRITE_SIZE hardware counters: what they
// report for this kernel, whose traffic is known, scales what they report for the SpMV kernels.
extern "C" int as_selftest_copy(int device, uint64_t bytes, int reps, float *ms_per_launch) {
  AS_API_BEGIN
  AS_CHECK(bytes >= 4096 && bytes % 16 == 0 && reps > 0, "bad size");
  std::string src =
      "extern \"C\" __global__ void __launch_bounds__(256) as_copy_words(const uint4 *__restrict__ in, uint4 *__restrict__ out, unsigned long long n)\n"
      "{\n  for (unsigned long long i = blockIdx.x * 256ull + threadIdx.x; i < n; i += gridDim.x * 256ull) out[i] = in[i];\n}\n";
  void *code = nullptr, *mod = nullptr, *fn = nullptr, *din = nullptr, *dout = nullptr, *e0 = nullptr, *e1 = nullptr;
  uint64_t n = 0;
  auto H = [](int r) { if (r != 0) throw asx::Error(as_hip_last_error()); };
  H(as_hip_compile(src.c_str(), "gfx950", nullptr, 0, &code, &n, nullptr));
  H(as_hip_init(device));
  H(as_hip_module_load(code, &mod));
  as_hip_free_host(code);
  H(as_hip_get_kernel(mod, "as_copy_words", &fn));
  H(as_hip_alloc(&din, bytes)); H(as_hip_alloc(&dout, bytes));
  H(as_hip_memset_async(din, 1, bytes, nullptr));
  H(as_hip_event_create(&e0)); H(as_hip_event_create(&e1));
  unsigned long long words = bytes / 16;
  void *args[] = {&din, &dout, &words};
  unsigned grid = (unsigned)std::min<unsigned long long>(1u << 20, (words + 255) / 256);
  H(as_hip_launch(fn, grid, 256, 0, nullptr, args));
  H(as_hip_event_record(e0, nullptr));
  for (int i = 0; i < reps; i++) H(as_hip_launch(fn, grid, 256, 0, nullptr, args));
  H(as_hip_event_record(e1, nullptr));
  H(as_hip_event_sync(e1));
  float ms = 0;
  H(as_hip_event_elapsed_ms(e0, e1, &ms));
  if (ms_per_launch) *ms_per_launch = ms / (float)reps;
  as_hip_event_destroy(e0); as_hip_event_destroy(e1);
  as_hip_free(din); as_hip_free(dout);
  as_hip_module_unload(mod);
  return 0;
  AS_API_END(-1)
}

// ---- search control and report text, one piece at a time (test hooks) --------------------------
extern "C" int64_t as_selftest_param_enumerator(int n, const long *low, const long *up, const long *step, long *out,
                                                uint64_t cap) {
  AS_API_BEGIN
  AS_CHECK(n > 0 && n <= 8 && low && up && step, "bad argument");
  std::vector<long> knob((size_t)n, 0);
  asx::ParamEnumerator e;
  for (int i = 0; i < n; i++) e.add(&knob[(size_t)i], low[i], up[i], step[i]);
  int64_t count = 0;
  while (e.next()) {
    for (int i = 0; i < n; i++)
      if (out && (uint64_t)(count * n + i) < cap) out[count * n + i] = knob[(size_t)i];
    count++;
  }
  return count;
  AS_API_END(-1)
}

extern "C" int as_selftest_search_strategy(uint64_t struggle_step_num, const float *gflops, int n, int *go) {
  AS_API_BEGIN
  AS_CHECK(gflops && go && n >= 0, "bad argument");
  asx::SearchStrategy s = asx::init_search_strategy(struggle_step_num, 1e9);
  for (int i = 0; i < n; i++) go[i] = asx::continue_search(s, gflops[i]) ? 1 : 0;
  return 0;
  AS_API_END(-1)
}

static int64_t put_text(const std::string &s, char *out, uint64_t cap) {
  if (out && cap) {
    strncpy(out, s.c_str(), cap - 1);
    out[cap - 1] = 0;
  }
  return (int64_t)s.size();
}

extern "C" int64_t as_strategy_report(int strategy, const long p[4], char *out, uint64_t cap) {
  AS_API_BEGIN
  AS_CHECK(p, "bad argument");
  asx::StrategyNode n = asx::make_strategy((asx::ParamStrategy)strategy, p[0], p[1], p[2], p[3]);
  return put_text(asx::convert_stategy_node_to_string(n), out, cap);
  AS_API_END(-1)
}

extern "C" int64_t as_graph_report(const long *desc, int64_t n_desc, int with_frame, float gflops, float time_ms, char *out,
                                   uint64_t cap) {
  AS_API_BEGIN
  AS_CHECK(desc && n_desc >= 2, "bad argument");
  int64_t at = 0;
  auto need = [&](int64_t more) { AS_CHECK(at + more <= n_desc, "the description of the graph ends early"); };
  auto node = [&]() {
    need(5);
    asx::StrategyNode n = asx::make_strategy((asx::ParamStrategy)desc[at], desc[at + 1], desc[at + 2], desc[at + 3], desc[at + 4]);
    if (n.strategy == asx::DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY) {
      n.in_nnz = (uint64_t)desc[at + 1];
      n.in_val_dtype = (asx::DType)desc[at + 2];
      n.in_col_index_max = (uint64_t)desc[at + 3];
      n.in_row_index_max = (uint64_t)desc[at + 4];
    }
    at += 5;
    return n;
  };
  asx::BestGraph g;
  need(1);
  for (long i = 0, n = desc[at++]; i < n; i++) g.dense.push_back(node());
  need(1);
  for (long s = 0, n_sub = desc[at++]; s < n_sub; s++) {
    asx::SubGraph sub;
    need(1);
    for (long i = 0, n = desc[at++]; i < n; i++) sub.nodes.push_back(node());
    need(4);
    sub.tpl.type = (asx::TemplateType)desc[at];
    sub.tpl.tblock_num = desc[at + 1];
    sub.tpl.thread_num_in_block = desc[at + 2];
    sub.tpl.thread_num_of_row_reduce = desc[at + 3];
    at += 4;
    g.subs.push_back(sub);
  }
  AS_CHECK(at == n_desc, "the description of the graph is longer than the graph");
  return put_text(with_frame ? asx::convert_search_result_to_string(gflops, time_ms, g) : asx::convert_graph_to_string(g), out, cap);
  AS_API_END(-1)
}

extern "C" int64_t as_template_node_report(int template_type, long tblock_num, long thread_num_in_block,
                                           long thread_num_of_row_reduce, char *out, uint64_t cap) {
  AS_API_BEGIN
  asx::TemplateNode n;
  n.type = (asx::TemplateType)template_type;
  n.tblock_num = tblock_num;
  n.thread_num_in_block = thread_num_in_block;
  n.thread_num_of_row_reduce = thread_num_of_row_reduce;
  return put_text(asx::convert_template_node_to_string(n), out, cap);
  AS_API_END(-1)
}
