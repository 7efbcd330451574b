// Optional per-kernel timing: when switched on (nmtg_trace_begin), every launch site brackets its
// kernel with two HIP events on the launch stream; nmtg_trace_end reads them back as
// (name, launches, total milliseconds). Off by default: one predictable branch per launch.
#pragma once
#include <hip/hip_runtime.h>

namespace nmtg {

bool trace_on();
void trace_open(const char* name, hipStream_t st, int* slot);
void trace_close(hipStream_t st, int slot);

struct TraceScope {
  hipStream_t st;
  int slot;
  TraceScope(const char* name, hipStream_t s) : st(s), slot(-1) {
    if (trace_on()) trace_open(name, s, &slot);
  }
  ~TraceScope() {
    if (slot >= 0) trace_close(st, slot);
  }
};

}  // namespace nmtg
