// ellm_attn_run_noalloc: the single-token attention step for callers that cannot
// allocate device memory (code under HIP graph capture, tight serving loops, harnesses
// that forbid hipMalloc).  Same kernel and split plan as ellm_attn_run /
// ellm_attn_run_ragged with position_interval == 1 (decode.hip); the split partials,
// cluster partials and arrival counters that a handle keeps in its own hipMalloc'd
// workspace live here in one file-scope device array instead.
//
// The array's name is a host-side stand-in, not a device address: host code only ever
// uses the address hipGetSymbolAddress returned for the device that is current, and each
// device holds its own copy of the array at its own address.
#include <hip/hip_runtime.h>

#include <mutex>

#include "../../include/ellm_attn.h"
#include "kernels.hpp"

namespace {

// Capacity of the static scratch: decode_plan.hpp (kStaticRows ...), where the host tests
// check it against every plan the planner returns.
constexpr size_t kRows = ellm::kStaticRows;
constexpr size_t kRows2 = ellm::kStaticRows2;
constexpr size_t kCounters = ellm::kStaticCounters;
constexpr size_t kOffMl = kRows * 128;
constexpr size_t kOffAcc2 = kOffMl + kRows * 2;
constexpr size_t kOffMl2 = kOffAcc2 + kRows2 * 128;
constexpr size_t kOffCounters = kOffMl2 + kRows2 * 2;
constexpr size_t kScratchFloats = kOffCounters + kCounters;   // 5,074,944 bytes
static_assert((kOffMl * 4) % 256 == 0 && (kOffAcc2 * 4) % 256 == 0 && (kOffMl2 * 4) % 256 == 0 &&
                  (kOffCounters * 4) % 256 == 0,
              "every table starts on a 256-byte boundary");

static __device__ __align__(256) float scratch[kScratchFloats];

constexpr int kMaxDevices = 64;
struct PerDevice {
  float* ptr;   // device address of this device's copy of `scratch`
  int n_cu;
  bool ready;
};
PerDevice g_devices[kMaxDevices];
std::mutex g_mutex;

// Arrival counters of the split merge, cleared ahead of the launch that counts in them.
// (A fill kernel, not hipMemsetAsync: the call may be recorded into a graph.)
__global__ void clear_counters_kernel(uint32_t* counters, uint32_t n) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0u;
}

// The current device's entry: its copy of the array's address and its compute-unit count.
// The steady-state cost is one hipGetDevice; the property query and the symbol lookup (a
// module load, which a stream capture in progress does not allow) run once per device, under
// the mutex, the first time a device is seen.
int prepare_current_device(const PerDevice** out) {
  int device = 0;
  const hipError_t got = hipGetDevice(&device);
  if (got != hipSuccess) {
    (void)hipGetLastError();
    return ellm::set_error(ELLM_ERR_NO_DEVICE, "hipGetDevice: %s", hipGetErrorString(got));
  }
  if (device < 0 || device >= kMaxDevices)
    return ellm::set_error(ELLM_ERR_UNSUPPORTED, "device %d: at most %d devices are tracked", device,
                           kMaxDevices);
  PerDevice& d = g_devices[device];
  if (__atomic_load_n(&d.ready, __ATOMIC_ACQUIRE)) {
    *out = &d;
    return ELLM_OK;
  }
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!d.ready) {
    int checked = 0, n_cu = 0;
    if (int st = ellm::current_gfx950_device(&checked, &n_cu)) return st;
    float* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return ellm::set_error(ELLM_ERR_HIP, "hipGetSymbolAddress(static scratch): %s",
                             hipGetErrorString(e));
    d.ptr = ptr;
    d.n_cu = n_cu;
    __atomic_store_n(&d.ready, true, __ATOMIC_RELEASE);
  }
  *out = &d;
  return ELLM_OK;
}

}  // namespace

// Called by the create functions (the nearest this library has to an init call) so that the
// symbol lookup has normally happened before the first ellm_attn_run_noalloc on a device.
void ellm::prepare_static_scratch() {
  const PerDevice* dev = nullptr;
  (void)prepare_current_device(&dev);   // a failure is reported by the call that needs the scratch
}

extern "C" {

int ellm_attn_run_noalloc(const ellm_attn_desc* desc, const uint32_t* positions, size_t position,
                          size_t batch_size, void* stream) {
  if (int st = ellm::validate_attn_desc(desc)) return st;
  if (ellm::attn_is_general(*desc))
    return ellm::set_error(ELLM_ERR_UNSUPPORTED, "head_size %zu / dtype %d: this entry point takes 128-wide 16-bit heads only",
                           desc->head_size, desc->dtype);
  if (batch_size == 0) return ELLM_OK;
  if (batch_size > desc->batch_size)
    return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu exceeds the capacity %zu", batch_size,
                           desc->batch_size);
  if (position >= desc->sequence_capacity)
    return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "position %zu is not below the sequence capacity %zu",
                           position, desc->sequence_capacity);
  const PerDevice* dev = nullptr;
  if (int st = prepare_current_device(&dev)) return st;

  ellm::AttnArgs a;
  ellm::attn_args_from_desc(*desc, &a);
  a.n_cu = (uint32_t)dev->n_cu;
  a.position_index = (uint32_t)position;
  a.position_interval = 1;
  a.batch = (uint32_t)batch_size;
  a.positions = positions;
  const ellm::DecodePlan plan =
      ellm::decode_plan((uint32_t)position + 1, a.batch, a.n_kv_heads, (uint32_t)dev->n_cu);
  a.split_len = plan.split_len;
  a.n_split = plan.n_split;
  if (plan.n_split > 1) {  // an unsplit launch touches no scratch at all
    const ellm::DecodeWorkspace room{kRows, kRows2, kCounters};
    const int over = ellm::decode_plan_exceeds(room, a.batch, a.n_q_heads, a.n_kv_heads, a.group, a.n_split);
    if (over) {
      const size_t n_cluster = (a.n_split + ellm::kPlanMergeFan - 1) / ellm::kPlanMergeFan;
      const size_t head_groups = (a.group + ellm::kPlanMaxHeadsPerGroup - 1) / ellm::kPlanMaxHeadsPerGroup;
      const char* what = over == 1 ? "split partial rows" : (over == 2 ? "cluster partial rows" : "arrival counters");
      const size_t need = over == 1 ? batch_size * a.n_q_heads * a.n_split
                                    : (over == 2 ? batch_size * a.n_q_heads * n_cluster
                                                 : batch_size * a.n_kv_heads * head_groups * (1 + n_cluster));
      const size_t have = over == 1 ? kRows : (over == 2 ? kRows2 : kCounters);
      return ellm::set_error(
          ELLM_ERR_OUT_OF_RANGE,
          "%zu sequences x %u query heads x %u splits need %zu %s; the static scratch holds %zu "
          "(use ellm_attn_create / ellm_attn_run, whose handle sizes its own workspace)",
          batch_size, a.n_q_heads, a.n_split, need, what, have);
    }
    float* base = dev->ptr;   // never the array's name: that is not a device address here
    a.ws_acc = base;
    a.ws_ml = base + kOffMl;
    a.ws2_acc = base + kOffAcc2;
    a.ws2_ml = base + kOffMl2;
    a.counters = (uint32_t*)(base + kOffCounters);
    // The array keeps the last call's contents.  Partials are written before they are read;
    // the counters must start at zero (they return to zero when a launch runs to its end,
    // but a launch that was cut short would leave them counting).
    hipLaunchKernelGGL(clear_counters_kernel, dim3((uint32_t)(kCounters / 256)), dim3(256), 0,
                       (hipStream_t)stream, a.counters, (uint32_t)kCounters);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
      return ellm::set_error(ELLM_ERR_HIP, "counter clear launch: %s", hipGetErrorString(e));
  }
  const hipError_t e = ellm::launch_decode(a, (hipStream_t)stream);
  if (e != hipSuccess)
    return ellm::set_error(ELLM_ERR_HIP, "single-token attention launch: %s", hipGetErrorString(e));
  return ELLM_OK;
}

}  // extern "C"
