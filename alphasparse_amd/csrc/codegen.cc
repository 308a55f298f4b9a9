// Source emission helpers shared by the kernel templates.
#include "device_facts.hpp"
#include "templates.hpp"

namespace asx {

std::string value_type_name(const Template &t) { return t.val_dtype == DOUBLE ? "double" : "float"; }
std::string y_row_type_name(const Template &) { return "unsigned int"; }

// Everything the generated kernels rely on.  Written for gfx950 only: 64-lane
// wavefronts, DPP row operations, hardware floating-point atomics.
std::string kernel_module_preamble() {
  return "#define AS_XCD_NUM " + std::to_string(kXcdNum) + "u\n" + R"SRC(
#define AS_WAVE 64
typedef unsigned int as_u32;
typedef unsigned long long as_u64;

template <typename T> __device__ __forceinline__ T as_ldnt(const T *p) { return __builtin_nontemporal_load(p); }
// y is written once and not read again by the kernel: a streaming store keeps it from displacing x in L2
template <typename T> __device__ __forceinline__ void as_stnt(T *p, T v) { __builtin_nontemporal_store(v, p); }

// The workgroup's barrier, with every LDS operation of the wavefront complete before it.  The plain barrier alone was
// compiled without the wait for outstanding LDS operations on one path into a barrier (a loop whose last iteration
// jumps over the block that held the wait): sums that one wavefront had added to LDS were read by another before
// they had landed.
__device__ __forceinline__ void as_barrier() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); __syncthreads(); }

__device__ __forceinline__ void as_atomic_add(float *p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void as_atomic_add(double *p, double v) { unsafeAtomicAdd(p, v); }

// Workgroups are handed to the 8 XCDs of the device in turn (workgroup i runs on XCD i % 8) and every XCD has
// its own L2.  A kernel whose neighbouring blocks read neighbouring pieces of x takes its block number from
// here instead of blockIdx.x: every XCD then works on a contiguous eighth of the blocks, and a line of x
// that two neighbouring blocks need is fetched into one L2, not two.  A permutation of [0, gridDim.x).
__device__ __forceinline__ unsigned int as_xcd_block_index(unsigned int b, unsigned int n) {
  return b < n / AS_XCD_NUM * AS_XCD_NUM ? (b % AS_XCD_NUM) * (n / AS_XCD_NUM) + b / AS_XCD_NUM : b;
}
__device__ __forceinline__ unsigned int as_xcd_block_index() { return as_xcd_block_index(blockIdx.x, gridDim.x); }

// One DPP move of a 32- or 64-bit value; lanes without a valid source read 0.
template <int CTRL, int ROW_MASK, int BANK_MASK> __device__ __forceinline__ float as_dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, BANK_MASK, false));
}
template <int CTRL, int ROW_MASK, int BANK_MASK> __device__ __forceinline__ double as_dpp(double v) {
  long long b = __double_as_longlong(v);
  int lo = (int)(b & 0xffffffffll), hi = (int)(b >> 32);
  lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, ROW_MASK, BANK_MASK, false);
  hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, ROW_MASK, BANK_MASK, false);
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// Sum over aligned groups of LANES lanes (LANES = 1,2,4,...,64).  After the
// call the LAST lane of every group holds the group's sum (for LANES <= 16 every
// lane of the group does).  row_ror:8 on a 16-lane row is its own inverse, so the
// sequence does not depend on the rotation direction.
template <int LANES, typename T> __device__ __forceinline__ T as_group_sum(T v) {
  if (LANES >= 2) v += as_dpp<0xb1, 0xf, 0xf>(v);    // quad_perm:[1,0,3,2]
  if (LANES >= 4) v += as_dpp<0x4e, 0xf, 0xf>(v);    // quad_perm:[2,3,0,1]
  if (LANES >= 8) v += as_dpp<0x141, 0xf, 0xf>(v);   // row_half_mirror: lane i <-> lane 7-i of its half row
  if (LANES >= 16) v += as_dpp<0x128, 0xf, 0xf>(v);  // row_ror:8
  if (LANES >= 32) v += as_dpp<0x142, 0xa, 0xf>(v);  // row_bcast:15 into rows 1,3
  if (LANES >= 64) v += as_dpp<0x143, 0xc, 0xf>(v);  // row_bcast:31 into rows 2,3
  return v;
}
template <typename T> __device__ __forceinline__ T as_wave_sum(T v) { return as_group_sum<64>(v); }

// Segmented sum along the lanes of a wavefront.  `key` is sorted along the lanes and never
// 0xffffffff; after the call every lane holds the sum of `v` over the lanes from the first lane
// of its run of equal keys up to itself, so the last lane of a run holds the run's sum.  Steps
// inside a 16-lane row shift by 1, 2, 4, 8; the two row_bcast steps carry the last lane of row 0
// (2) into row 1 (3) and lane 31 into rows 2 and 3 -- with sorted keys a lane that matches the
// carried key continues that run.  Lanes without a source lane compare against 0xffffffff.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ unsigned int as_dpp_key(unsigned int k) {
  return (unsigned int)__builtin_amdgcn_update_dpp((int)0xffffffffu, (int)k, CTRL, ROW_MASK, 0xf, false);
}
template <int CTRL, int ROW_MASK, typename T> __device__ __forceinline__ T as_segmented_step(unsigned int key, T v) {
  const unsigned int k2 = as_dpp_key<CTRL, ROW_MASK>(key);
  const T v2 = as_dpp<CTRL, ROW_MASK, 0xf>(v);
  return k2 == key ? v + v2 : v;
}
template <typename T> __device__ __forceinline__ T as_wave_segmented_sum(unsigned int key, T v) {
  v = as_segmented_step<0x111, 0xf>(key, v);  // row_shr:1
  v = as_segmented_step<0x112, 0xf>(key, v);  // row_shr:2
  v = as_segmented_step<0x114, 0xf>(key, v);  // row_shr:4
  v = as_segmented_step<0x118, 0xf>(key, v);  // row_shr:8
  v = as_segmented_step<0x142, 0xa>(key, v);  // row_bcast:15 into rows 1,3
  v = as_segmented_step<0x143, 0xc>(key, v);  // row_bcast:31 into rows 2,3
  return v;
}
// true in the last lane of every run of equal keys (wave_shl:1 reads the next lane's key)
__device__ __forceinline__ bool as_is_segment_tail(unsigned int key) { return as_dpp_key<0x130, 0xf>(key) != key; }

// Sum into LDS shared by the lanes of one workgroup.
template <typename T> __device__ __forceinline__ void as_lds_add(T *p, T v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// Same sums through ds_bpermute shuffles; used to cross-check the DPP path.
template <int LANES, typename T> __device__ __forceinline__ T as_group_sum_shfl(T v) {
  for (int o = LANES / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
)SRC";
}

std::string kernel_signature(const Template &t) { return kernel_signature(t, std::string()); }

std::string kernel_signature(const Template &t, const std::string &p) {
  std::string s;
  for (auto &a : t.arrays)
    if (a.passed()) s += std::string("const ") + dtype_c_name(a.a.dt) + " *__restrict__ " + p + a.name + ", ";
  std::string vt = value_type_name(t);
  s += "const " + vt + " *__restrict__ " + p + "val_arr, const " + std::string(dtype_c_name(t.col_index_arr.dt)) +
       " *__restrict__ " + p + "col_index_arr, const " + vt + " *__restrict__ " + p + "device_x_arr, " + vt + " *__restrict__ " + p + "device_y_arr";
  if (t.scratch_bytes) s += ", unsigned int *__restrict__ " + p + "scratch_arr";
  return s;
}

std::string kernel_arguments(const Template &t, const std::string &p) {
  std::string s;
  for (auto &a : t.arrays)
    if (a.passed()) s += p + a.name + ", ";
  s += p + "val_arr, " + p + "col_index_arr, " + p + "device_x_arr, " + p + "device_y_arr";
  if (t.scratch_bytes) s += ", " + p + "scratch_arr";
  return s;
}

std::string kernel_trips_function_name(const Template &t) { return "spmv_" + std::to_string(t.sub) + "_trips"; }

bool carried_place_is_passed(const Template &guest) { return guest.arr("y_row_index").passed(); }

std::string carried_finish_signature(const Template &host) {
  if (!host.carried) return std::string();
  const Template &g = *host.carried;
  std::string s = ", " + value_type_name(g) + " *__restrict__ carried_sum";
  if (carried_place_is_passed(g))
    s += std::string(", const ") + dtype_c_name(g.arr("y_row_index").a.dt) + " *__restrict__ carried_place";
  return s + ", unsigned int carried_rows";
}

std::string carried_finish_prologue(const Template &host, uint64_t threads) {
  if (!host.carried) return "  const unsigned int as_block = blockIdx.x, as_grid = gridDim.x;\n";
  const Template &g = *host.carried;
  const TArr &place = g.arr("y_row_index");
  const std::string GB = std::to_string(host.carried_blocks) + "u", B = std::to_string(threads) + "u";
  // The rows of the strip before this one wait in its scratch vector for their places in y: a few workgroups of
  // this kernel move them there (and leave the vector cleared) while the others start on their own work, instead
  // of a kernel of its own between the two strips -- a launch and a chain of two memory round trips that nothing
  // overlapped.  A whole number of eights of workgroups, so that the others keep their XCDs.
  std::string s;
  s += "  if (blockIdx.x < " + GB + ")\n  {\n";
  s += "    for (unsigned int sub_row = blockIdx.x * " + B + " + threadIdx.x; sub_row < carried_rows; sub_row += " + GB + " * " + B + ")\n    {\n";
  s += "      const " + value_type_name(g) + " sum = carried_sum[sub_row];\n";
  s += "      carried_sum[sub_row] = 0;\n";
  s += "      unsigned int global_row_index;\n";
  if (place.c.active()) {
    s += "      " + code_of_arr_read(place.c, "global_row_index", "sub_row");
    if (place.c.type != BRANCH_COMPRESS) s += ";\n";
  } else {
    s += "      global_row_index = carried_place[sub_row];\n";
  }
  s += "      as_stnt(device_y_arr + global_row_index, sum);\n";
  s += "    }\n    return;\n  }\n";
  s += "  const unsigned int as_block = blockIdx.x - " + GB + ", as_grid = gridDim.x - " + GB + ";\n";
  return s;
}

std::string code_of_meta_read(const Template &t, const std::string &arr, const std::string &var,
                              const std::string &idx) {
  const TArr &a = t.arr(arr);
  if (!a.c.active()) return var + " = " + arr + "[" + idx + "];\n";
  std::string s = code_of_arr_read(a.c, var, idx);
  if (a.c.type != BRANCH_COMPRESS) s += ";\n";
  return s;
}

}  // namespace asx
