// What the format builders and the search need to know about the GPU: how many compute units share the work,
// how much LDS a workgroup may take, and the cache that decides whether x can stay close.  The values are those of
// an MI355X (gfx950, all eight XCDs as one device) until a GPU has been asked; read_device_facts replaces the CU
// count and the LDS size by what the runtime reports and refuses a GPU of another architecture: the kernels are
// written for gfx950 only.
#pragma once
#include <cstdint>

namespace asx {

// gfx950: 64-lane wavefronts, workgroups are handed to the XCDs in turn, every XCD has its own L2 cache
constexpr uint64_t kWaveLanes = 64;
constexpr uint64_t kXcdNum = 8;
constexpr uint64_t kL2BytesPerXcd = 4ull << 20;

struct DeviceFacts {
  uint64_t cu_num = 256;        // compute units of the device
  uint64_t lds_bytes = 163840;  // LDS one workgroup may use (a CU's whole LDS on gfx950)
  bool from_device = false;     // read from a GPU (or set by the caller) rather than assumed
};

const DeviceFacts &device_facts();
// Bytes of x that a kernel with a slice of x in LDS keeps there: four fifths of a workgroup's LDS (128 KB of 160).
uint64_t x_slice_bytes();
// Asks GPU `device` once per process (later calls return at once); throws for a GPU that is not a gfx950.
void read_device_facts(int device);
// For callers that build formats for a GPU they cannot ask (another partition mode, tests): 0 keeps a value.
void set_device_facts(uint64_t cu_num, uint64_t lds_bytes);
// back to the MI355X values, to be read from a GPU again at the next upload or search
void reset_device_facts();

}  // namespace asx
