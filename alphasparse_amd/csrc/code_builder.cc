#include <mutex>
#include <unordered_map>
#include "code_builder.hpp"

#include <cstring>

#include "device_facts.hpp"
#include "hip_layer.h"

namespace asx {

static const size_t kMaxKernelArgs = 64;

#define HIPL(call)                                                                      \
  do {                                                                                  \
    if ((call) != 0) throw Error(std::string(#call) + " failed: " + as_hip_last_error()); \
  } while (0)

std::vector<uint8_t> narrow_bytes(const IArr &a) {
  int w = dtype_size(a.dt);
  AS_CHECK(w > 0, "array has no element type");
  if (w < 8) {
    const uint64_t limit = (1ull << (8 * w)) - 1;
    for (size_t i = 0; i < a.size(); i++)
      if (a[i] > limit) throw Error("narrow_bytes: a value does not fit the element type chosen for its array");
  }
  std::vector<uint8_t> out(a.size() * (size_t)w);
  switch (w) {
    case 1: for (size_t i = 0; i < a.size(); i++) out[i] = (uint8_t)a[i]; break;
    case 2: { auto *p = (uint16_t *)out.data(); for (size_t i = 0; i < a.size(); i++) p[i] = (uint16_t)a[i]; break; }
    case 4: { auto *p = (uint32_t *)out.data(); for (size_t i = 0; i < a.size(); i++) p[i] = (uint32_t)a[i]; break; }
    default: memcpy(out.data(), a.v.data(), out.size());
  }
  return out;
}

std::vector<uint8_t> narrow_values(const ValVec &v, DType dt) {
  if (dt == DOUBLE) {
    std::vector<uint8_t> out(v.size() * 8);
    memcpy(out.data(), v.data(), out.size());
    return out;
  }
  std::vector<uint8_t> out(v.size() * 4);
  float *p = (float *)out.data();
  for (size_t i = 0; i < v.size(); i++) p[i] = (float)v[i];
  return out;
}

std::unique_ptr<Builder> init_code_builder(const Matrix &m) {
  AS_CHECK(m.is_compressed && !m.items.empty(), "matrix is not compressed");
  auto b = std::make_unique<Builder>();
  b->matrix = &m;
  b->rows = m.y_rows;  // length of y
  b->rows_compacted = m.rows_compacted;
  b->cols = m.cols;
  b->origin_nnz = m.origin_nnz;
  b->val_dtype = m.val_dtype;
  b->subs.resize(m.items.size());
  return b;
}

void invalidate_module(Builder &b) {
  b.source.clear();
  b.code.clear();
  b.module_stale = true;
}
static void invalidate(Builder &b) { invalidate_module(b); }

static void free_sub_arrays(SubKernel &k) {
  for (auto &m : k.meta) as_hip_free(m.ptr);
  k.meta.clear();
  if (k.val.ptr) as_hip_free(k.val.ptr);
  if (k.col.ptr) as_hip_free(k.col.ptr);
  if (k.scratch.ptr) as_hip_free(k.scratch.ptr);
  k.val = k.col = k.scratch = DeviceBuf();
  k.uploaded = false;
}

void add_template_to_builder(Builder &b, uint64_t sub, TemplateType type) {
  AS_CHECK(b.matrix != nullptr && sub < b.subs.size(), "sub-matrix id out of range");
  if (b.subs[sub].uploaded) {
    as_hip_device_sync();
    free_sub_arrays(b.subs[sub]);
  }
  b.subs[sub].tpl = init_template(type, *b.matrix, sub);
  b.subs[sub].tpl->y_needs_clear = template_needs_cleared_y(*b.subs[sub].tpl, *b.matrix, sub);
  invalidate(b);
}

void remove_template_from_builder(Builder &b, uint64_t sub) {
  AS_CHECK(sub < b.subs.size(), "sub-matrix id out of range");
  if (b.subs[sub].uploaded) {
    as_hip_device_sync();
    free_sub_arrays(b.subs[sub]);
  }
  b.subs[sub].tpl.reset();
  b.subs[sub].fn = nullptr;
  invalidate(b);
}

bool compress_template_in_builder(Builder &b, uint64_t sub) {
  AS_CHECK(sub < b.subs.size() && b.subs[sub].tpl, "sub-matrix has no template");
  AS_CHECK(!b.subs[sub].uploaded, "compress a template before it is uploaded");
  try_all_compress(*b.subs[sub].tpl);
  invalidate(b);
  for (auto &a : b.subs[sub].tpl->arrays)
    if (a.c.active()) return true;
  return false;
}

bool set_relative_columns(Builder &b, uint64_t sub) {
  AS_CHECK(sub < b.subs.size() && b.subs[sub].tpl, "sub-matrix has no template");
  if (!make_columns_relative(*b.subs[sub].tpl)) return false;
  if (b.subs[sub].uploaded) {
    as_hip_device_sync();
    free_sub_arrays(b.subs[sub]);
    b.subs[sub].uploaded = false;
  }
  invalidate(b);
  return true;
}

bool set_diagonal_columns(Builder &b, uint64_t sub) {
  AS_CHECK(sub < b.subs.size() && b.subs[sub].tpl, "sub-matrix has no template");
  if (!make_columns_diagonal(*b.subs[sub].tpl)) return false;
  if (b.subs[sub].uploaded) {
    as_hip_device_sync();
    free_sub_arrays(b.subs[sub]);
    b.subs[sub].uploaded = false;
  }
  invalidate(b);
  return true;
}

bool set_row_ownership(Builder &b, uint64_t sub) {
  AS_CHECK(b.matrix != nullptr && sub < b.subs.size() && b.subs[sub].tpl, "sub-matrix has no template");
  Template &old = *b.subs[sub].tpl;
  if (old.type != SHARED_MEMORY_TILE_TEMPLATE || old.own_rows) return false;
  std::unique_ptr<Template> t = init_tile_template_variant(*b.matrix, sub, old.col_runs, true);
  if (!t) return false;
  // the zero-valued elements that close lanes where a row of a group is missing from a slice must stay few
  if ((double)t->val_arr.size() > 1.05 * (double)old.val_arr.size()) return false;
  try_all_compress(*t);
  t->y_needs_clear = template_needs_cleared_y(*t, *b.matrix, sub);
  t->thread_num_in_block = old.thread_num_in_block;
  set_default_launch(*t);
  if (b.subs[sub].uploaded) {
    as_hip_device_sync();
    free_sub_arrays(b.subs[sub]);
    b.subs[sub].uploaded = false;
  }
  b.subs[sub].tpl = std::move(t);
  invalidate(b);
  return true;
}

bool set_row_blocks(Builder &b, uint64_t sub, uint64_t rows_per_block) {
  AS_CHECK(b.matrix != nullptr && sub < b.subs.size() && b.subs[sub].tpl, "sub-matrix has no template");
  AS_CHECK(rows_per_block >= 2 && rows_per_block <= 4, "blocks of 2, 3 or 4 rows");
  Template &old = *b.subs[sub].tpl;
  if (old.type != SHARED_MEMORY_TILE_TEMPLATE || !old.own_rows || old.row_block != 1) return false;
  std::unique_ptr<Template> t = init_tile_template_variant(*b.matrix, sub, old.col_runs, true, rows_per_block);
  if (!t) return false;
  try_all_compress(*t);
  t->y_needs_clear = template_needs_cleared_y(*t, *b.matrix, sub);
  t->thread_num_in_block = old.thread_num_in_block;
  set_default_launch(*t);
  if (b.subs[sub].uploaded) {
    as_hip_device_sync();
    free_sub_arrays(b.subs[sub]);
    b.subs[sub].uploaded = false;
  }
  b.subs[sub].tpl = std::move(t);
  invalidate(b);
  return true;
}

bool add_tile_template_variant_to_builder(Builder &b, uint64_t sub, bool column_runs_if_shorter, bool own_rows, uint64_t row_block) {
  AS_CHECK(b.matrix != nullptr && sub < b.subs.size(), "sub-matrix id out of range");
  // column runs where set_column_runs would take them: the stream must get at least 2 % shorter, lane-closing
  // padding included; counted in one pass before anything is built
  const double vs = (double)dtype_size(b.matrix->val_dtype);
  const CompressedBlock &cb = *b.matrix->items[sub].cb;
  const double plain = (double)cb.read_index[0]->index_arr.v.size() * (vs + 2.5);
  const bool runs = column_runs_if_shorter && (double)tile_column_run_stream_estimate(*b.matrix, sub) * (vs + 1.625) <= 0.98 * plain;
  std::unique_ptr<Template> t = init_tile_template_variant(*b.matrix, sub, runs, own_rows, row_block);
  if (!t) return false;
  try_all_compress(*t);
  t->y_needs_clear = template_needs_cleared_y(*t, *b.matrix, sub);
  set_default_launch(*t);
  if (b.subs[sub].uploaded) {
    as_hip_device_sync();
    free_sub_arrays(b.subs[sub]);
    b.subs[sub].uploaded = false;
  }
  b.subs[sub].tpl = std::move(t);
  invalidate(b);
  return true;
}

bool set_column_runs(Builder &b, uint64_t sub) {
  AS_CHECK(b.matrix != nullptr && sub < b.subs.size() && b.subs[sub].tpl, "sub-matrix has no template");
  Template &old = *b.subs[sub].tpl;
  if (old.type != SHARED_MEMORY_TILE_TEMPLATE || old.col_runs) return false;
  // worth it when the element stream gets shorter: the padding that closes lanes must not eat the 7 bytes per
  // lane that the columns save.  Counted first (one pass over the columns), so that a matrix of scattered columns,
  // where every element is a run of its own, is turned down before the form is built.
  const double vs = (double)dtype_size(old.val_dtype);
  const double before = (double)old.val_arr.size() * (vs + 2.5);
  if ((double)tile_column_run_stream_estimate(*b.matrix, sub) * (vs + 1.625) > 0.98 * before) return false;
  std::unique_ptr<Template> t = init_tile_template_variant(*b.matrix, sub, true, old.own_rows, old.row_block);
  if (!t) return false;
  const double after = (double)t->val_arr.size() * (vs + 1.625);
  if (after > 0.98 * before) return false;
  try_all_compress(*t);
  t->y_needs_clear = template_needs_cleared_y(*t, *b.matrix, sub);
  t->thread_num_in_block = old.thread_num_in_block;
  set_default_launch(*t);
  if (b.subs[sub].uploaded) {
    as_hip_device_sync();
    free_sub_arrays(b.subs[sub]);
    b.subs[sub].uploaded = false;
  }
  b.subs[sub].tpl = std::move(t);
  invalidate(b);
  return true;
}

int64_t assign_finish_carriers(const Builder &b, uint64_t sub) {
  int64_t carrier_of_sub = -1;
  const SubKernel *before = nullptr;
  for (auto &k : b.subs) {
    if (!k.tpl) continue;
    k.tpl->carried = nullptr;
    k.tpl->carried_blocks = 0;
    k.tpl->fused_trips = nullptr;
    // the strip before leaves its rows in a scratch vector for a finish kernel, and this one starts with a kernel
    // that does not touch y: the two are independent, and the rows of the strip before are this kernel's to move
    if (b.serial_launch && b.carry_finish && before && before->tpl->type == SHARED_MEMORY_TILE_TEMPLATE &&
        before->tpl->finish_tblock_num && before->tpl->scratch_bytes && k.tpl->type == SHARED_MEMORY_PRODUCT_BIN_TEMPLATE) {
      k.tpl->carried = before->tpl.get();
      // With workgroups of the same size the two strips' first kernels become one launch as well: every workgroup
      // runs a trip of the strip before and then trips of this one, so the tail of the one and the start of the other
      // overlap CU by CU instead of meeting at a kernel boundary; the carried rows then wait for this strip's SECOND
      // kernel, which starts when every trip is done.
      if (b.fuse_launches && before->tpl->thread_num_in_block == k.tpl->thread_num_in_block) k.tpl->fused_trips = before->tpl.get();
      const uint64_t rows = before->tpl->sc("sub_rows");
      const uint64_t threads = std::max<uint64_t>(64, k.tpl->fused_trips ? k.tpl->finish_thread_num : k.tpl->thread_num_in_block);
      k.tpl->carried_blocks = std::min<uint64_t>(256, ((rows + threads - 1) / threads + 7) / 8 * 8);
      if (k.tpl->fused_trips) {
        // The second kernel's own workgroups are all on the device at once where they fit (two of 1024 threads per
        // CU): carriers on top of them would be a second round of workgroups, a tail of a few microseconds behind
        // the first.  As many carriers as still fit the first round, at least eight; each then moves more rows.
        const uint64_t per_cu = std::max<uint64_t>(1, std::min<uint64_t>(2048 / std::max<uint64_t>(64, k.tpl->finish_thread_num),
                                                                       device_facts().lds_bytes / std::max<uint64_t>(1, k.tpl->finish_lds_bytes)));
        const uint64_t room = device_facts().cu_num * per_cu;
        if (k.tpl->finish_tblock_num <= room && k.tpl->finish_tblock_num + k.tpl->carried_blocks > room)
          k.tpl->carried_blocks = std::max<uint64_t>(8, (room - k.tpl->finish_tblock_num) / 8 * 8);
      }
      if (before->tpl->sub == sub) carrier_of_sub = (int64_t)k.tpl->sub;
    }
    before = &k;
  }
  return carrier_of_sub;
}

std::string build_module_source(const Builder &b) {
  assign_finish_carriers(b);
  std::string s = kernel_module_preamble();
  s += "extern \"C\" __global__ void as_zero_words(unsigned int *p, unsigned long long n)\n{\n"
       "  for (unsigned long long i = blockIdx.x * (unsigned long long)blockDim.x + threadIdx.x; i < n;\n"
       "       i += (unsigned long long)gridDim.x * blockDim.x) p[i] = 0u;\n}\n";
  size_t n = 0;
  for (auto &k : b.subs) {
    if (!k.tpl) continue;  // partial execution: only the sub-matrices that have a template
    s += "\n// " + std::string(convert_template_type_to_string(k.tpl->type)) + "\n" + code_of_template_kernal(*k.tpl);
    n++;
  }
  AS_CHECK(n > 0, "no sub-matrix has a template");
  return s;
}

// Code objects of this process by module source.  The search compiles the same text more than once (the
// winner of a strategy is rebuilt for the longer re-measurement and again for the caller), and a compilation
// costs far more than a lookup.  Bounded: emptied when it holds more than kCodeCacheBytes.
namespace {
const size_t kCodeCacheBytes = 256u << 20;
std::mutex g_code_cache_mutex;
std::unordered_map<std::string, std::vector<char>> g_code_cache;
size_t g_code_cache_bytes = 0;
uint64_t g_code_cache_hits = 0;
}  // namespace

void code_cache_stats(uint64_t &entries, uint64_t &hits) {
  std::lock_guard<std::mutex> lock(g_code_cache_mutex);
  entries = g_code_cache.size();
  hits = g_code_cache_hits;
}

void compile_builder(Builder &b) {
  if (!b.code.empty()) return;
  b.source = build_module_source(b);
  {
    std::lock_guard<std::mutex> lock(g_code_cache_mutex);
    auto hit = g_code_cache.find(b.source);
    if (hit != g_code_cache.end()) {
      b.code = hit->second;
      g_code_cache_hits++;
      b.compile_log.clear();
      return;
    }
  }
  void *code = nullptr;
  uint64_t n = 0;
  char *log = nullptr;
  int r = as_hip_compile(b.source.c_str(), "gfx950", nullptr, 0, &code, &n, &log);
  b.compile_log = log ? log : "";
  if (log) as_hip_free_host(log);
  if (r != 0) throw Error(std::string("kernel compilation failed: ") + as_hip_last_error());
  b.code.assign((char *)code, (char *)code + n);
  as_hip_free_host(code);
  std::lock_guard<std::mutex> lock(g_code_cache_mutex);
  if (g_code_cache_bytes + b.source.size() + b.code.size() > kCodeCacheBytes) {
    g_code_cache.clear();
    g_code_cache_bytes = 0;
  }
  if (g_code_cache.emplace(b.source, b.code).second) g_code_cache_bytes += b.source.size() + b.code.size();
}

static DeviceBuf upload(const std::vector<uint8_t> &bytes) {
  DeviceBuf d;
  d.bytes = bytes.size();
  HIPL(as_hip_alloc(&d.ptr, d.bytes));
  if (d.bytes) HIPL(as_hip_h2d(d.ptr, bytes.data(), d.bytes));
  return d;
}

static void ensure_module(Builder &b) {
  if (!b.module_stale && b.module) return;
  compile_builder(b);
  if (b.module) {
    as_hip_device_sync();
    as_hip_module_unload(b.module);
    b.module = nullptr;
  }
  HIPL(as_hip_module_load(b.code.data(), &b.module));
  HIPL(as_hip_get_kernel(b.module, "as_zero_words", &b.zero_fn));
  for (auto &k : b.subs) {
    if (!k.tpl) continue;
    k.fn = k.finish_fn = nullptr;
    if (k.tpl->type == EMPTY_TEMPLATE) continue;  // no kernel
    std::string name = "spmv_" + std::to_string(k.tpl->sub);
    HIPL(as_hip_get_kernel(b.module, name.c_str(), &k.fn));
    k.finish_fn = nullptr;
    if (k.tpl->finish_tblock_num) HIPL(as_hip_get_kernel(b.module, (name + "_finish").c_str(), &k.finish_fn));
  }
  b.module_stale = false;
}

void load_and_upload(Builder &b, int device) {
  if (!b.device_ready) {
    HIPL(as_hip_init(device));
    read_device_facts(device);
    HIPL(as_hip_stream_create(&b.main_stream));
    HIPL(as_hip_event_create(&b.start_ev));
    HIPL(as_hip_event_create(&b.t0));
    HIPL(as_hip_event_create(&b.t1));
    size_t vs = (size_t)dtype_size(b.val_dtype);
    HIPL(as_hip_alloc(&b.x.ptr, b.cols * vs));
    b.x.bytes = b.cols * vs;
    HIPL(as_hip_alloc(&b.y.ptr, b.rows * vs));
    b.y.bytes = b.rows * vs;
    // the static scratch array of this GPU, for the entry point that allocates nothing: looked up here, once
    // (a failed lookup only disables that entry point, which then says so)
    if (as_hip_static_scratch(device, &b.static_scratch, &b.static_scratch_bytes) != 0) {
      b.static_scratch = nullptr;
      b.static_scratch_bytes = 0;
    }
    b.device_ready = true;
  }
  ensure_module(b);
  for (auto &k : b.subs) {
    if (!k.tpl || k.uploaded) continue;
    for (auto &a : k.tpl->arrays)
      if (a.passed()) k.meta.push_back(upload(narrow_bytes(a.a)));
    k.val = upload(narrow_values(k.tpl->val_arr, k.tpl->val_dtype));
    k.col = upload(narrow_bytes(k.tpl->col_index_arr));
    if (k.tpl->scratch_bytes) k.scratch = upload(std::vector<uint8_t>(k.tpl->scratch_bytes, 0));
    if (!k.stream) {
      HIPL(as_hip_stream_create(&k.stream));
      HIPL(as_hip_event_create(&k.done));
    }
    k.uploaded = true;
  }
}

// Launches the kernels of every active sub-matrix.  static_scratch != nullptr: the kernels' scratch arrays are
// 256-byte aligned pieces of that memory (in sub-matrix order) instead of the builder's own allocations.
static void launch_kernels(Builder &b, void *stream, const void *x_dev, void *y_dev, unsigned char *static_scratch = nullptr) {
  size_t active = 0;
  auto skipped = [&](const SubKernel &k) { return !k.tpl || (b.only_sub >= 0 && &k != &b.subs[(size_t)b.only_sub]); };
  for (auto &k : b.subs) active += !skipped(k);
  bool multi = active > 1 && !b.serial_launch;
  if (multi) HIPL(as_hip_event_record(b.start_ev, stream));
  uint64_t scratch_offset = 0;
  const SubKernel *before = nullptr;  // the sub-matrix with a template in front of the current one
  void *scratch_before = nullptr;
  for (size_t idx = 0; idx < b.subs.size(); idx++) {
    SubKernel &k = b.subs[idx];
    void *scratch_ptr = k.scratch.ptr;
    if (k.tpl && k.tpl->scratch_bytes && static_scratch) {
      scratch_ptr = static_scratch + scratch_offset;
      scratch_offset += (k.tpl->scratch_bytes + 255) / 256 * 256;
    }
    const SubKernel *guest = before;
    void *guest_scratch = scratch_before;
    if (k.tpl) {
      before = &k;
      scratch_before = scratch_ptr;
    }
    if (skipped(k)) continue;
    if (k.tpl->type == EMPTY_TEMPLATE) continue;  // nothing to launch: its rows of y are the clear's
    AS_CHECK(k.uploaded && k.fn, "a template was changed after upload: call upload again");
    // kernel arguments: passed metadata arrays, val, col, x, y, scratch -- a fixed-size list, nothing allocated
    void *ptrs[kMaxKernelArgs], *first_args[kMaxKernelArgs], *finish_args[kMaxKernelArgs];
    size_t n = 0;
    auto push_arrays = [&](const SubKernel &from, void *from_scratch) {
      AS_CHECK(n + from.meta.size() + 8 <= kMaxKernelArgs, "too many kernel arguments");
      for (auto &m : from.meta) ptrs[n++] = m.ptr;
      ptrs[n++] = from.val.ptr;
      ptrs[n++] = from.col.ptr;
      ptrs[n++] = (void *)x_dev;
      ptrs[n++] = y_dev;
      if (from.tpl->scratch_bytes) ptrs[n++] = from_scratch;
    };
    push_arrays(k, scratch_ptr);
    const size_t n_own = n;
    for (size_t i = 0; i < n_own; i++) first_args[i] = finish_args[i] = &ptrs[i];
    size_t n_first = n_own, n_finish = n_own;
    // A kernel that carries the finish of the strip before it takes that strip's scratch vector, its places in y and
    // its number of rows behind its own arguments -- 0 rows when this strip is launched alone.  With a fused launch
    // the first kernel takes all arrays of the strip before instead (and a flag: 0 when this strip is launched alone),
    // and the second kernel carries.
    unsigned int carried_rows = 0, fused_on = 0;
    if (k.tpl->carried) {
      AS_CHECK(guest && guest->tpl.get() == k.tpl->carried && guest->uploaded, "a template was changed after upload: call upload again");
      void **carrier_args = k.tpl->fused_trips ? finish_args : first_args;
      size_t &n_carrier = k.tpl->fused_trips ? n_finish : n_first;
      ptrs[n] = guest_scratch;
      carrier_args[n_carrier++] = &ptrs[n++];
      if (carried_place_is_passed(*guest->tpl)) {
        size_t at = 0;
        for (auto &a : guest->tpl->arrays) {
          if (a.name == "y_row_index") break;
          at += a.passed();
        }
        ptrs[n] = guest->meta[at].ptr;
        carrier_args[n_carrier++] = &ptrs[n++];
      }
      if (b.only_sub < 0) carried_rows = (unsigned int)guest->tpl->sc("sub_rows");
      carrier_args[n_carrier++] = &carried_rows;
      if (k.tpl->fused_trips) {
        const size_t guest_first = n;
        push_arrays(*guest, guest_scratch);
        for (size_t i = guest_first; i < n; i++) first_args[n_first++] = &ptrs[i];
        fused_on = b.only_sub < 0 ? 1u : 0u;
        first_args[n_first++] = &fused_on;
      }
    }
    // ... and the strip before it then launches no finish kernel of its own (with a fused launch: no kernel at all)
    bool finish_is_carried = false, trips_are_fused = false;
    if (b.only_sub < 0)
      for (size_t j = idx + 1; j < b.subs.size(); j++)
        if (b.subs[j].tpl) {
          finish_is_carried = b.subs[j].tpl->carried == k.tpl.get();
          trips_are_fused = b.subs[j].tpl->fused_trips == k.tpl.get();
          break;
        }
    void *s = multi ? k.stream : stream;
    if (multi) HIPL(as_hip_stream_wait_event(s, b.start_ev));
    if (b.only_pass != 2 && !trips_are_fused) {
      uint64_t grid = k.tpl->tblock_num, lds = k.tpl->dynamic_lds_bytes;
      if (k.tpl->fused_trips && fused_on) {
        grid = std::max(grid, guest->tpl->tblock_num);
        lds = std::max(lds, guest->tpl->dynamic_lds_bytes);
      } else if (!k.tpl->fused_trips) {
        grid += k.tpl->carried_blocks;
      }
      HIPL(as_hip_launch(k.fn, (unsigned)grid, (unsigned)k.tpl->thread_num_in_block, (unsigned)lds, s, first_args));
    }
    if (k.tpl->finish_tblock_num && b.only_pass != 1 && !finish_is_carried) {
      AS_CHECK(k.finish_fn, "a template was changed after upload: call upload again");
      HIPL(as_hip_launch(k.finish_fn, (unsigned)(k.tpl->finish_tblock_num + (k.tpl->fused_trips ? k.tpl->carried_blocks : 0)),
                         (unsigned)k.tpl->finish_thread_num, (unsigned)k.tpl->finish_lds_bytes, s, finish_args));
    }
    if (multi) {
      HIPL(as_hip_event_record(k.done, s));
      HIPL(as_hip_stream_wait_event(stream, k.done));
    }
  }
}

static void zero_words(Builder &b, void *stream, void *p, unsigned long long words) {
  void *args[] = {&p, &words};
  unsigned grid = (unsigned)std::min<unsigned long long>(4096, (words + 255) / 256);
  HIPL(as_hip_launch(b.zero_fn, std::max(1u, grid), 256, 0, stream, args));
}

static void zero_y(Builder &b, void *stream, void *y_dev) {
  zero_words(b, stream, y_dev, (unsigned long long)b.rows * dtype_size(b.val_dtype) / 4);
}

void clear_scratch(Builder &b, uint64_t sub) {
  AS_CHECK(b.device_ready && sub < b.subs.size() && b.subs[sub].tpl, "sub-matrix has no template on the device");
  SubKernel &k = b.subs[sub];
  if (!k.tpl->scratch_bytes || !k.scratch.ptr) return;
  zero_words(b, b.main_stream, k.scratch.ptr, (k.tpl->scratch_bytes + 3) / 4);
  HIPL(as_hip_stream_sync(b.main_stream));
}

bool y_needs_clear(const Builder &b) {
  // rows taken out by remove_empty_rows keep their place in y and are stored by no kernel
  if (b.rows_compacted) return true;
  for (auto &k : b.subs)
    if (!k.tpl || k.tpl->y_needs_clear) return true;  // a sub-matrix without kernel leaves its rows unwritten
  return false;
}

static void check_launch_shapes(const Builder &b) {
  for (auto &k : b.subs) {
    if (!k.tpl) continue;
    AS_CHECK(k.tpl->tblock_num > 0 && k.tpl->tblock_num < (1ull << 31), "bad grid size");
    AS_CHECK(k.tpl->thread_num_in_block > 0 && k.tpl->thread_num_in_block <= 1024 &&
                 k.tpl->thread_num_in_block % 64 == 0, "threads per block must be a multiple of 64, at most 1024");
  }
}

void launch_spmv(Builder &b, const void *x_dev, void *y_dev, void *stream) {
  AS_CHECK(b.device_ready, "builder is not on the device");
  ensure_module(b);
  check_launch_shapes(b);
  if (y_needs_clear(b)) zero_y(b, stream, y_dev);
  launch_kernels(b, stream, x_dev, y_dev);
}
void launch_spmv(Builder &b, const void *x_dev, void *y_dev) { launch_spmv(b, x_dev, y_dev, b.main_stream); }

uint64_t static_scratch_need(const Builder &b) {
  uint64_t need = 0;
  for (auto &k : b.subs)
    if (k.tpl && k.tpl->scratch_bytes) need += (k.tpl->scratch_bytes + 255) / 256 * 256;
  return need;
}

void launch_spmv_no_alloc(Builder &b, const void *x_dev, void *y_dev) { launch_spmv_no_alloc(b, x_dev, y_dev, b.main_stream); }
void launch_spmv_no_alloc(Builder &b, const void *x_dev, void *y_dev, void *stream) {
  AS_CHECK(b.device_ready && b.module && !b.module_stale, "builder is not on the device: call upload first (this entry point loads nothing)");
  for (auto &k : b.subs) AS_CHECK(!k.tpl || k.uploaded, "a template was changed after upload: call upload again");
  check_launch_shapes(b);
  const uint64_t need = static_scratch_need(b);
  AS_CHECK(need == 0 || b.static_scratch, "no static scratch array on this device (its address could not be looked up at upload): use as_builder_spmv_device");
  AS_CHECK(need <= b.static_scratch_bytes,
           "the kernels of this graph need " + std::to_string(need) + " bytes of scratch, the static scratch array holds " +
               std::to_string(b.static_scratch_bytes) + ": use as_builder_spmv_device");
  unsigned char *base = (unsigned char *)b.static_scratch;
  // Every call on this GPU shares the array, which holds what the last call left: the pieces whose kernels add
  // into them are cleared by the fill kernel (no memset node, so the sequence can be captured)
  uint64_t offset = 0;
  for (auto &k : b.subs) {
    if (!k.tpl || !k.tpl->scratch_bytes) continue;
    if (k.tpl->scratch_starts_zero) zero_words(b, stream, base + offset, (k.tpl->scratch_bytes + 3) / 4);
    offset += (k.tpl->scratch_bytes + 255) / 256 * 256;
  }
  if (y_needs_clear(b)) zero_y(b, stream, y_dev);
  launch_kernels(b, stream, x_dev, y_dev, base ? base : nullptr);
}

void spmv_host(Builder &b, const void *x_host, void *y_host) {
  AS_CHECK(b.device_ready, "builder is not on the device");
  HIPL(as_hip_h2d(b.x.ptr, x_host, b.x.bytes));
  launch_spmv(b, b.x.ptr, b.y.ptr);
  HIPL(as_hip_stream_sync(b.main_stream));
  HIPL(as_hip_d2h(y_host, b.y.ptr, b.y.bytes));
}

void time_spmv(Builder &b, uint64_t reps, bool sync_each, float &time_ms, float &gflops) {
  AS_CHECK(b.device_ready && reps > 0, "builder is not on the device");
  ensure_module(b);
  check_launch_shapes(b);
  // The timed step is the product call: what launch_spmv issues, the clear of y included where the graph needs
  // it.  Measurements of one sub-matrix's kernels alone (only_sub) are kernel times: y is cleared once, before.
  const bool clear_each = b.only_sub < 0 && y_needs_clear(b);
  if (b.only_sub >= 0) {
    zero_y(b, b.main_stream, b.y.ptr);
    HIPL(as_hip_stream_sync(b.main_stream));
  }
  HIPL(as_hip_event_record(b.t0, b.main_stream));
  for (uint64_t r = 0; r < reps; r++) {
    if (clear_each) zero_y(b, b.main_stream, b.y.ptr);
    launch_kernels(b, b.main_stream, b.x.ptr, b.y.ptr);
    if (sync_each) HIPL(as_hip_stream_sync(b.main_stream));
  }
  HIPL(as_hip_event_record(b.t1, b.main_stream));
  HIPL(as_hip_event_sync(b.t1));
  HIPL(as_hip_event_elapsed_ms(b.t0, b.t1, &time_ms));
  uint64_t nnz = 0;
  for (auto &k : b.subs)
    if (k.tpl && (b.only_sub < 0 || &k == &b.subs[(size_t)b.only_sub])) nnz += k.tpl->origin_nnz;
  gflops = (float)(2.0 * (double)nnz * (double)reps / ((double)time_ms * 1e6));
}

uint64_t builder_algorithmic_bytes(const Builder &b) {
  uint64_t vs = (uint64_t)dtype_size(b.val_dtype), bytes = b.cols * vs + b.rows * vs;
  for (auto &k : b.subs)
    if (k.tpl) bytes += template_format_bytes(*k.tpl);
  if (y_needs_clear(b)) bytes += b.rows * vs;  // the clear writes y once more
  return bytes;
}

void release_device(Builder &b) {
  if (!b.device_ready) return;
  as_hip_device_sync();
  for (auto &k : b.subs) {
    free_sub_arrays(k);
    if (k.stream) as_hip_stream_destroy(k.stream);
    if (k.done) as_hip_event_destroy(k.done);
    k.stream = k.done = nullptr;
    k.fn = nullptr;
  }
  if (b.x.ptr) as_hip_free(b.x.ptr);
  if (b.y.ptr) as_hip_free(b.y.ptr);
  b.x = b.y = DeviceBuf();
  for (void **e : {&b.start_ev, &b.t0, &b.t1})
    if (*e) { as_hip_event_destroy(*e); *e = nullptr; }
  if (b.main_stream) as_hip_stream_destroy(b.main_stream);
  b.main_stream = nullptr;
  if (b.module) as_hip_module_unload(b.module);
  b.module = nullptr;
  b.device_ready = false;
}

Builder::~Builder() { release_device(*this); }

}  // namespace asx
