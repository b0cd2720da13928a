// Error plumbing shared by every entry point: the last error text is kept per host thread.
#include <stdarg.h>
#include <string.h>

#include "common.hpp"

namespace gptoss {

int trace_set(void *const *start, void *const *stop, int n);
int trace_count();
const char *trace_name(int i);

static thread_local char g_last_error[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

const char *last_error() { return g_last_error; }

struct TraceState {
  hipEvent_t *start = nullptr, *stop = nullptr;
  int capacity = 0, count = 0;
  const char *names[4096];
};
static thread_local TraceState g_trace;

TraceScope::TraceScope(const char *name, hipStream_t s) : slot(-1), stream(s) {
  TraceState &t = g_trace;
  if (t.start == nullptr || t.count >= t.capacity || t.count >= 4096) return;
  slot = t.count++;
  t.names[slot] = name;
  (void)hipEventRecord(t.start[slot], stream);
}

TraceScope::~TraceScope() {
  if (slot >= 0) (void)hipEventRecord(g_trace.stop[slot], stream);
}

int trace_set(void *const *start, void *const *stop, int n) {
  g_trace.start = (hipEvent_t *)start;
  g_trace.stop = (hipEvent_t *)stop;
  g_trace.capacity = (start && stop) ? n : 0;
  g_trace.count = 0;
  if (!(start && stop)) g_trace.start = g_trace.stop = nullptr;
  return GPTOSS_OK;
}
int trace_count() { return g_trace.count; }
const char *trace_name(int i) { return (i >= 0 && i < g_trace.count) ? g_trace.names[i] : ""; }

}  // namespace gptoss

extern "C" const char *gptoss_last_error_string(void) { return gptoss::last_error(); }
extern "C" int gptoss_abi_version(void) { return 101; }
extern "C" int gptoss_trace_set(void *const *start_events, void *const *stop_events, int n) {
  if (n < 0) return gptoss::fail(GPTOSS_ERR_DIM, "trace_set: negative count");
  return gptoss::trace_set(start_events, stop_events, n);
}
extern "C" int gptoss_trace_count(void) { return gptoss::trace_count(); }
extern "C" const char *gptoss_trace_name(int i) { return gptoss::trace_name(i); }
