// Test build only: stands in for fairring_amd/csrc/ksum_kernels.hip when the
// pipeline is compiled against the fake HIP runtime. The "kernel" is a plain
// fp32 fold run as one unit of work on the fake stream, so the choreography
// around it (ordering, slot reuse, carry chains) decides whether results come
// out right. fp32 only.
#include <hip/hip_runtime.h>

#include <vector>

#include "../../fairring_amd/csrc/ksum_kernels.h"
#include "../../include/fairring_hip.h"

namespace frg {

int64_t elementSize(int dtype) {
  switch (dtype) {
    case FRG_F32:
    case FRG_I32:
      return 4;
    case FRG_BF16:
    case FRG_F16:
      return 2;
    case FRG_F64:
    case FRG_I64:
      return 8;
    case FRG_U8:
    case FRG_I8:
      return 1;
    default:
      return 0;
  }
}

bool isFloating(int dtype) {
  return dtype == FRG_F32 || dtype == FRG_BF16 || dtype == FRG_F16 || dtype == FRG_F64;
}

void setTuning(int) {}

namespace {

struct Job {
  float* out;
  std::vector<const float*> in;
  int64_t n;
  int op;
  int scaleMode;
  float scale;
  bool carry;
};

void runJob(void* p) {
  Job* j = static_cast<Job*>(p);
  for (int64_t i = 0; i < j->n; ++i) {
    size_t k = 0;
    float acc = j->carry ? j->out[i] : j->in[k++][i];
    for (; k < j->in.size(); ++k) {
      const float b = j->in[k][i];
      if (j->op == FRG_SUM) {
        acc = acc + b;
      } else {
        acc = (acc != acc) ? acc : ((b != b) ? b : (acc > b ? acc : b));
      }
    }
    if (j->scaleMode == FRG_SCALE_MUL) acc = acc * j->scale;
    if (j->scaleMode == FRG_SCALE_DIV) acc = acc / j->scale;
    j->out[i] = acc;
  }
  delete j;
}

}  // namespace

int launchReduce(const ReduceArgs& a, hipStream_t stream, std::string* err) {
  auto fail = [&](int code, const char* msg) {
    if (err) *err = msg;
    return code;
  };
  if (a.dtype != FRG_F32) return fail(FRG_ERR_UNSUPPORTED, "host test build reduces fp32 only");
  if (a.op != FRG_SUM && a.op != FRG_MAX) return fail(FRG_ERR_UNSUPPORTED, "unsupported op");
  if (a.K < 1 || a.K > kMaxContribsPerLaunch) return fail(FRG_ERR_INVALID, "K out of range");
  if (a.n < 0) return fail(FRG_ERR_INVALID, "negative element count");
  if (a.n == 0) return FRG_OK;
  if (a.out == nullptr || a.contribs == nullptr) return fail(FRG_ERR_INVALID, "null pointer");
  Job* j = new Job{static_cast<float*>(a.out), {}, a.n, a.op, a.scale_mode, a.scale, a.carry};
  for (int k = 0; k < a.K; ++k) j->in.push_back(static_cast<const float*>(a.contribs[k]));
  if (a.startEvent) hipEventRecord(a.startEvent, stream);
  fake_hip_enqueue(stream, &runJob, j);
  if (a.stopEvent) hipEventRecord(a.stopEvent, stream);
  return FRG_OK;
}

}  // namespace frg
