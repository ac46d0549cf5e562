// Optional per-kernel timing with HIP events on the launch stream (off by default; zero cost
// when off).  When on, every launcher brackets its kernel with two events; report() waits for
// the stream, turns the pairs into durations and aggregates them per kernel tag together with
// the algorithmic flops and bytes the launcher declared.
#include <map>
#include <sstream>
#include <vector>

#include "common.hpp"

namespace nncv_hip {

namespace {
struct Rec {
  std::string name;
  double flops, bytes;
  hipEvent_t e0, e1;
};
struct State {
  bool on = false;
  std::vector<Rec> recs;
  std::vector<hipEvent_t> pool;
};
State& st() {
  static State s;
  return s;
}
hipEvent_t take_event() {
  State& s = st();
  if (!s.pool.empty()) {
    hipEvent_t e = s.pool.back();
    s.pool.pop_back();
    return e;
  }
  hipEvent_t e;
  NNCV_HIP_CHECK(hipEventCreate(&e));
  return e;
}
}  // namespace

bool profiler_enabled() { return st().on; }
void profiler_enable(bool on) { st().on = on; }

ProfScope::ProfScope(const char* name, double flops, double bytes, hipStream_t s) : s_(s), on_(st().on) {
  if (!on_) return;
  Rec r{name, flops, bytes, take_event(), take_event()};
  NNCV_HIP_CHECK(hipEventRecord(r.e0, s));
  st().recs.push_back(r);
}
ProfScope::~ProfScope() {
  if (!on_) return;
  (void)hipEventRecord(st().recs.back().e1, s_);
}

std::string profiler_report() {
  State& s = st();
  struct Agg { long long n = 0; double ms = 0, flops = 0, bytes = 0; };
  std::map<std::string, Agg> agg;
  for (Rec& r : s.recs) {
    NNCV_HIP_CHECK(hipEventSynchronize(r.e1));
    float ms = 0;
    NNCV_HIP_CHECK(hipEventElapsedTime(&ms, r.e0, r.e1));
    Agg& a = agg[r.name];
    a.n += 1; a.ms += ms; a.flops += r.flops; a.bytes += r.bytes;
    s.pool.push_back(r.e0);
    s.pool.push_back(r.e1);
  }
  s.recs.clear();
  std::ostringstream os;
  os.precision(9);
  os << "{";
  bool first = true;
  for (auto& kv : agg) {
    if (!first) os << ", ";
    first = false;
    os << "\"" << kv.first << "\": {\"launches\": " << kv.second.n << ", \"ms\": " << kv.second.ms
       << ", \"flops\": " << kv.second.flops << ", \"bytes\": " << kv.second.bytes << "}";
  }
  os << "}";
  return os.str();
}

}  // namespace nncv_hip
