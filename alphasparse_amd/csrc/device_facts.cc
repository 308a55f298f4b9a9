#include "device_facts.hpp"

#include <cstring>
#include <mutex>

#include "as_types.hpp"
#include "hip_layer.h"

namespace asx {

namespace {
DeviceFacts g_facts;
std::mutex g_facts_mutex;
}  // namespace

const DeviceFacts &device_facts() { return g_facts; }
uint64_t x_slice_bytes() { return g_facts.lds_bytes / 5 * 4; }

void read_device_facts(int device) {
  std::lock_guard<std::mutex> lock(g_facts_mutex);
  if (g_facts.from_device) return;
  char name[256] = {0};
  int cus = 0, wave = 0;
  uint64_t lds = 0, mem = 0;
  if (as_hip_device_info(device, name, (int)sizeof(name), &cus, &wave, &lds, &mem) != 0) throw Error(as_hip_last_error());
  AS_CHECK(strstr(name, "gfx950") != nullptr && wave == (int)kWaveLanes,
           std::string("the kernels of this library are written for gfx950 (64-lane wavefronts); the device is ") + name);
  AS_CHECK(cus > 0 && lds >= 65536, "the device reports no compute units or less than 64 KB of LDS per workgroup");
  g_facts.cu_num = (uint64_t)cus;
  g_facts.lds_bytes = lds;
  g_facts.from_device = true;
}

void set_device_facts(uint64_t cu_num, uint64_t lds_bytes) {
  std::lock_guard<std::mutex> lock(g_facts_mutex);
  if (cu_num) g_facts.cu_num = cu_num;
  if (lds_bytes) g_facts.lds_bytes = lds_bytes;
  g_facts.from_device = true;
}


void reset_device_facts() {
  std::lock_guard<std::mutex> lock(g_facts_mutex);
  g_facts = DeviceFacts();
}

}  // namespace asx
