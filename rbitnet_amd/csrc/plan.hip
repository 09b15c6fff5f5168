// Recorded steps: the launches of one step of a model, noted once while the host code of the
// step runs (Python: the parts' forward functions), issued again from here as often as a step of
// the same shape comes back, with one call from the host in place of some hundreds.  A plan holds
// closures over the entry points' arguments; the pointers among them stay the caller's business
// (the memory they name must be the same memory at every replay: the caller keeps the step's
// buffers in a pool of their own).  What changes between the steps of one shape (token ids,
// positions, page tables, the rows asked for) lies in device buffers that the kernels read.
//
// Recording is per thread; a plan is replayed by one thread at a time.
#include <vector>

#include "api.h"
#include "common.h"

struct RbPlan {
  std::vector<std::function<int(void*)>> calls;
};

static thread_local RbPlan* g_recording = nullptr;
static thread_local int g_depth = 0;        // entry points running on this thread, one inside the other

RbPlanScope::RbPlanScope() { ++g_depth; }
RbPlanScope::~RbPlanScope() { --g_depth; }
bool rb_plan_wants_call(void) { return g_recording != nullptr && g_depth == 1; }
void rb_plan_note(std::function<int(void*)> call) { g_recording->calls.push_back(std::move(call)); }

extern "C" void* rb_plan_begin(void) {
  if (g_recording) {
    rb_set_error("rb_plan_begin: a plan is being recorded on this thread already");
    return nullptr;
  }
  g_recording = new RbPlan();
  return g_recording;
}

extern "C" int rb_plan_end(void* plan) {
  RB_REQUIRE(plan != nullptr && plan == g_recording, "rb_plan_end: this plan is not the one being recorded");
  g_recording = nullptr;
  return 0;
}

extern "C" int rb_plan_calls(void* plan) { return plan ? (int)((RbPlan*)plan)->calls.size() : 0; }

extern "C" int rb_plan_replay(void* plan, void* stream) {
  RB_REQUIRE(plan != nullptr, "rb_plan_replay: no plan");
  RB_REQUIRE(plan != g_recording, "rb_plan_replay: the plan is still being recorded");
  for (auto& call : ((RbPlan*)plan)->calls) {
    const int rc = call(stream);
    if (rc) return rc;
  }
  return 0;
}

extern "C" void rb_plan_free(void* plan) {
  if (plan == g_recording) g_recording = nullptr;
  delete (RbPlan*)plan;
}
