// Named ranges around the host-layer phases, for profiler timelines (`rocprofv3
// --marker-trace`): the MI355X counterpart of the NVTX ranges the reference's benchmarks put
// around their sampling steps (examples/randomwalk/randomwalk_fused_bench.py:37-39).  With no
// profiler attached a range is two calls into a library that has no subscriber.
#pragma once

#ifndef GS_NO_RANGES
#include <rocprofiler-sdk-roctx/roctx.h>
#endif

namespace gs {

class Range {
 public:
#ifndef GS_NO_RANGES
  explicit Range(const char* name) { roctxRangePushA(name); }
  ~Range() { roctxRangePop(); }
#else
  explicit Range(const char*) {}
#endif
  Range(const Range&) = delete;
  Range& operator=(const Range&) = delete;
};

}  // namespace gs
