// The drop-in body for the reference's part_execute_code_builder (executor.hpp:12-17), as a maintainer of the
// reference would write it over the C ABI, compiled as a program: a 5-point stencil goes through COMPRESS, row
// padding and the ELL template, the wrapper runs it with the reference's own default launch count, and the
// program prints what came back.  Written against include/alphasparse_amd.h only.
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "alphasparse_amd.h"

// ---- the documented wrapper, unchanged ---------------------------------------------------------
bool part_execute_code_builder(as_builder *b, std::vector<int> sub_matrix_id_vec, float &time_ms, float &gflops,
                               std::string /*execute_path*/, std::string /*data_path*/, bool /*store_data*/) {
  std::vector<int64_t> ids(sub_matrix_id_vec.begin(), sub_matrix_id_vec.end());
  if (as_builder_compile(b) != 0 || as_builder_upload(b, 0) != 0) return false;
  return as_part_execute_code_builder(b, ids.data(), ids.size(), /*repeat=*/0, &time_ms, &gflops) == 0;
}
// -------------------------------------------------------------------------------------------------

static int fail(const char *what) {
  fprintf(stderr, "%s: %s\n", what, as_last_error());
  return 1;
}

int main(int argc, char **argv) {
  const uint64_t g = argc > 1 ? strtoull(argv[1], nullptr, 10) : 1024;  // grid side
  std::vector<uint64_t> row, col;
  std::vector<double> val;
  for (uint64_t i = 0; i < g; i++)
    for (uint64_t j = 0; j < g; j++) {
      const uint64_t r = i * g + j;
      auto put = [&](uint64_t c, double v) { row.push_back(r); col.push_back(c); val.push_back(v); };
      if (i > 0) put(r - g, -1.0);
      if (j > 0) put(r - 1, -1.0);
      put(r, 4.0);
      if (j + 1 < g) put(r + 1, -1.0);
      if (i + 1 < g) put(r + g, -1.0);
    }
  as_matrix *m = as_matrix_from_coo(g * g, g * g, row.size(), row.data(), col.data(), val.data(), AS_FLOAT, 64);
  if (!m) return fail("as_matrix_from_coo");
  long pad[2] = {64, 1};
  if (as_execute_node(m, AS_COMPRESS, -1, nullptr, 0, nullptr, 0, nullptr, 0) != 0 ||
      as_execute_node(m, AS_COMPRESSED_ROW_PADDING, 0, pad, 2, nullptr, 0, nullptr, 0) != 0 ||
      as_execute_node(m, AS_COMPRESSED_THREAD_LEVEL_ROW_DIV, 0, nullptr, 0, nullptr, 0, nullptr, 0) != 0 ||
      as_complete_blocking(m, 0) != 0)
    return fail("operator graph");
  as_builder *b = as_builder_create(m);
  if (!b || as_builder_set_template(b, 0, AS_DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS) != 0) return fail("template");
  // padded elements of the sub-matrix = what the default launch count is sized by
  const int64_t padded = as_template_get_f64(b, 0, nullptr, 0);
  float time_ms = 0, gflops = 0;
  if (!part_execute_code_builder(b, std::vector<int>{0}, time_ms, gflops, "", "", false)) return fail("part_execute_code_builder");
  printf("nnz:%llu\npadded_nnz:%lld\ntime_ms:%g\ngflops:%g\n", (unsigned long long)row.size(), (long long)padded, time_ms, gflops);
  as_builder_free(b);
  as_matrix_free(m);
  return 0;
}
