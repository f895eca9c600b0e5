// Decoding step of the MVPA forward on a workspace that lives inside the library, for callers that
// cannot allocate device memory (code under HIP graph capture, tight serving loops).
//
// The split last-step launch of mvpa_forward cuts the cached key steps into runs and passes the
// runs' partial outputs and log-sum-exps to a merge kernel through a workspace the caller brings
// (mvpa_fwd_args.split_ws).  Here that workspace is a file-scope device array: each GPU the library
// runs on holds its own copy of it (MVPA_STATIC_WS_BYTES) until the process ends.  The host-side
// name of the array is not a device address; the address on the current device is looked up once
// per device and that pointer is what the kernels receive, exactly as they receive split_ws.
#include <atomic>

#include "mvpa_common.h"

static __device__ __align__(256) unsigned char scratch[MVPA_STATIC_WS_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];   // device address of `scratch`, per device

// Address of this device's copy of the array; nullptr if the runtime cannot tell.
void* scratch_on_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p) return p;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
  g_scratch_ptr[dev].store(p, std::memory_order_release);   // racing first calls store the same value
  return p;
}
}  // namespace

extern "C" size_t mvpa_static_ws_bytes(void) { return (size_t)MVPA_STATIC_WS_BYTES; }

// Set-up call: looks the array's address on the current device up and keeps it, so that no later
// call has to ask the runtime for it - in particular not the first call under stream capture.
extern "C" int mvpa_static_ws_init(void) { return scratch_on_current_device() ? MVPA_OK : MVPA_ERR_LAUNCH; }

extern "C" int mvpa_forward_last_step_static(const mvpa_fwd_args* a, void* stream) {
  if (!a) return MVPA_ERR_NULL;
  if (a->struct_size != sizeof(mvpa_fwd_args)) return MVPA_ERR_STRUCT;
  if (!(a->flags & MVPA_FLAG_LAST_STEP) || a->n_split <= 1) return MVPA_ERR_UNSUPPORTED;
  if (a->B <= 0 || a->H <= 0 || a->C <= 0 || a->Dh <= 0) return MVPA_ERR_SHAPE;
  if (mvpa_split_ws_bytes(a) > (size_t)MVPA_STATIC_WS_BYTES) return MVPA_ERR_WS_SIZE;
  mvpa_fwd_args b = *a;
  b.kernel = MVPA_KERNEL_MFMA;              // the only kernel that splits the key steps
  b.split_ws = (void*)(uintptr_t)256;       // placeholder so that validation sees a workspace
  const int st = mvpa_validate(&b);
  if (st != MVPA_OK) return st;
  if (!(b.flags & MVPA_FLAG_CONTENT)) return MVPA_ERR_UNSUPPORTED;   // launched unsplit: no workspace in play
  void* ws = scratch_on_current_device();
  if (!ws) return MVPA_ERR_LAUNCH;
  b.split_ws = ws;
  // Every run writes all of its rows before the merge kernel reads them, so nothing in the array
  // has to start at zero; what the last call left there is overwritten or never read.
  return mvpa_forward(&b, stream);
}
