// Tail splitting: which items of a launch are cut into parts (see SplitPlan in fba_kernels.h).
#include <cstdlib>
#include <mutex>

#include "fba_kernels.h"

namespace fba {

namespace {

// Compute units of the current device (looked up once per device).
int compute_units() {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static int cache[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  std::lock_guard<std::mutex> lock(mu);
  if (cache[dev] == 0) {
    int n = 0;
    cache[dev] = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256;
  }
  return cache[dev];
}

}  // namespace

int device_compute_units() { return compute_units(); }

namespace {
constexpr int kQueueBytes = 256;
__global__ void queue_reset_kernel(int* queue) { queue[threadIdx.x] = 0; }
}  // namespace

bool claims_wanted(int items_per_xcd, int total_work, int wgs_per_cu) {
  const char* e = getenv("FBA_CLAIM_WORK");
  const bool off = e != nullptr && e[0] == '0';
  (void)items_per_xcd;  // either mapping deals grid index i to XCD i % 8, which is all a claim relies on
  return !off && total_work >= 4 * compute_units() * wgs_per_cu;
}

int* work_queue_in(void* ws, int64_t ws_bytes, int64_t partial_bytes) {
  if (ws == nullptr) return nullptr;
  const int64_t off = (ws_bytes - kQueueBytes) & ~(int64_t)15;
  if (off < partial_bytes) return nullptr;
  return reinterpret_cast<int*>(static_cast<char*>(ws) + off);
}

hipError_t launch_queue_reset(int* queue, hipStream_t stream) {
  hipLaunchKernelGGL(queue_reset_kernel, dim3(1), dim3(kQueueBytes / 4), 0, stream, queue);
  return hipGetLastError();
}

// The hardware hands work-groups to free slots in index order.  With n items on s slots the last n % s items form a
// partial round; when that round would fill at most half of the slots, each of its items is cut into floor(s / (n % s))
// parts (at most 8), so that the parts fill the slots once and take 1 / parts of a round.  Launches smaller than the
// machine (n < s) are split the same way.
SplitPlan plan_split(int num_items, int wgs_per_cu, int64_t slot_bytes, void* ws, int64_t ws_bytes) {
  SplitPlan plan{nullptr, num_items, 1, 0};
  if (ws == nullptr || num_items <= 0) return plan;
  int slots = compute_units() * wgs_per_cu;
  if (slots > kSplitMaxSlots) slots = kSplitMaxSlots;
  const int rest = num_items % slots;
  if (rest == 0 || 2 * rest > slots) return plan;
  int parts = slots / rest;
  if (parts > 8) parts = 8;
  while (parts >= 2 && (int64_t)rest * parts * slot_bytes > ws_bytes) --parts;
  if (parts < 2) return plan;
  plan.ws = static_cast<float*>(ws);
  plan.first = num_items - rest;
  plan.parts = parts;
  return plan;
}

}  // namespace fba
