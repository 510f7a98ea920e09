// frg_reduce_slice_static: the K-way reduction of one slice for any number of
// contributions on the caller's stream, for callers that cannot allocate (a
// stream under HIP graph capture, a serving loop, a harness that forbids
// hipMalloc). frg_allreduce chains the launches of more than 64 contributions
// through a scratch buffer that the context allocates (schedule_resident.cc,
// chainThroughScratch); here the same chain runs through an array that is part
// of the library's device code, so the call allocates nothing.
#include <hip/hip_runtime.h>

#include <mutex>
#include <string>
#include <vector>

#include "../../include/fairring_hip.h"
#include "ksum_kernels.h"
#include "pipeline.h"

namespace {

// The partial result of a chain, in fp32 accumulators for bf16 / fp16 sums, in
// the storage type otherwise. Every GPU the library runs on holds its own copy
// until the process ends. 16 bytes to spare: placeInScratch() moves the start
// by up to that to keep the vector variant of the kernel.
constexpr int64_t kScratchBytes = FRG_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes + 256];

// In host code `scratch` is only a handle for the runtime: the array's address
// on a device is what hipGetSymbolAddress reports with that device current,
// asked once per device and kept.
constexpr int kMaxDevices = 64;
std::mutex gScratchMu;
char* gScratchPtr[kMaxDevices];

int scratchOnCurrentDevice(char** ptr, std::string* err) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    (void)hipGetLastError();
    *err = "no current HIP device (or more than 64 of them)";
    return FRG_ERR_HIP;
  }
  std::lock_guard<std::mutex> g(gScratchMu);
  if (gScratchPtr[device] == nullptr) {
    void* p = nullptr;
    const hipError_t r = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (r != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      *err = std::string("hipGetSymbolAddress of the static scratch failed: ") +
             hipGetErrorString(r);
      return FRG_ERR_HIP;
    }
    gScratchPtr[device] = static_cast<char*>(p);
  }
  *ptr = gScratchPtr[device];
  return FRG_OK;
}

int fail(int code, const std::string& msg) {
  frg::setLastError(msg);
  return code;
}

}  // namespace

namespace frg {

// Looks the array up for `device` ahead of the first call (Context::create does
// so for its device, so that a caller that creates a context first never meets
// the runtime's lazy set-up inside a capture). Failures are left to the call.
void prepareStaticScratch(int device) {
  int prev = 0;
  if (hipGetDevice(&prev) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  if (prev != device && hipSetDevice(device) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  char* p = nullptr;
  std::string err;
  (void)scratchOnCurrentDevice(&p, &err);
  if (prev != device) (void)hipSetDevice(prev);
}

}  // namespace frg

extern "C" int frg_reduce_slice_static(void* out, const void* const* contribs, int K, int64_t n,
                                       int dtype, int op, int scale_mode, float scale,
                                       void* stream) {
  using frg::kMaxContribsPerLaunch;
  const int64_t elsize = frg::elementSize(dtype);
  if (elsize == 0) return fail(FRG_ERR_UNSUPPORTED, "unsupported dtype");
  if (K < 1 || contribs == nullptr) {
    return fail(FRG_ERR_INVALID, "at least one contribution is required");
  }
  if (K > FRG_STATIC_MAX_CONTRIBUTIONS) {
    return fail(FRG_ERR_INVALID, "at most " + std::to_string(FRG_STATIC_MAX_CONTRIBUTIONS) +
                                     " contributions, got " + std::to_string(K));
  }
  if (n < 0) return fail(FRG_ERR_INVALID, "negative element count");
  hipStream_t s = static_cast<hipStream_t>(stream);
  std::string err;
  if (K <= kMaxContribsPerLaunch) {
    // one launch: nothing to carry, no scratch
    frg::ReduceArgs a;
    a.out = out;
    a.contribs = contribs;
    a.K = K;
    a.n = n;
    a.dtype = dtype;
    a.op = op;
    a.scale_mode = scale_mode;
    a.scale = scale;
    const int rc = frg::launchReduce(a, s, &err);
    return rc == FRG_OK ? FRG_OK : fail(rc, err);
  }
  if (n == 0) return FRG_OK;
  if (out == nullptr) return fail(FRG_ERR_INVALID, "null output");
  // A chain of launches. bf16 / fp16 sums keep their partial sums in fp32
  // between the launches (one rounding, at the end, like a single launch); a
  // result reduced in place into a contribution that only a later launch reads
  // must not land there early. Both park the partial result in the scratch;
  // every other chain carries it in `out` itself, exactly.
  const bool acc = op == FRG_SUM && (dtype == FRG_BF16 || dtype == FRG_F16);
  bool lateAlias = false;
  for (int k = kMaxContribsPerLaunch; k < K; ++k) {
    if (contribs[k] == out) lateAlias = true;
  }
  char* park = nullptr;
  if (acc || lateAlias) {
    const int64_t need = n * (acc ? 4 : elsize);
    if (need > kScratchBytes) {
      return fail(FRG_ERR_INVALID,
                  "a chain over " + std::to_string(K) + " contributions of this type parks " +
                      std::to_string(acc ? 4 : elsize) + " bytes per element in the static "
                      "scratch of " + std::to_string(kScratchBytes) + " bytes: at most " +
                      std::to_string(kScratchBytes / (acc ? 4 : elsize)) + " elements, got " +
                      std::to_string(n) + " (cut the slice, or use frg_allreduce)");
    }
    char* base = nullptr;
    const int rc = scratchOnCurrentDevice(&base, &err);
    if (rc != FRG_OK) return fail(rc, err);
    park = frg::placeInScratch(base, acc ? contribs[0] : out, acc, elsize);
  }
  for (int k0 = 0; k0 < K; k0 += kMaxContribsPerLaunch) {
    const int kn = K - k0 < kMaxContribsPerLaunch ? K - k0 : kMaxContribsPerLaunch;
    const bool last = k0 + kn == K;
    frg::ReduceArgs a;
    a.out = (park != nullptr && !last) ? static_cast<void*>(park) : out;
    a.out_acc = acc && !last;
    a.contribs = contribs + k0;
    a.K = kn;
    a.n = n;
    a.dtype = dtype;
    a.op = op;
    // a post-scale goes on the last launch only, a pre-scale on every one
    a.scale_mode = (last || scale_mode >= FRG_SCALE_PRE_MUL) ? scale_mode : FRG_SCALE_NONE;
    a.scale = scale;
    a.carry = k0 > 0;
    a.carry_src = park;  // null: carried in `out`
    a.carry_acc = acc;
    const int rc = frg::launchReduce(a, s, &err);
    if (rc != FRG_OK) return fail(rc, err);
  }
  return FRG_OK;
}
