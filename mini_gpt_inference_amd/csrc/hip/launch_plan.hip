// A step's launches as data: the model's forward pass is a sequence of launcher calls whose
// arguments (buffer addresses in the workspace and the step's arena, sizes, constants) are the same
// for every step of the same shape.  The Python side decides them once, when a shape is first
// seen, and records them here; every later step of that shape is one call into this file, which
// makes the launches from C++ (also under HIP graph capture).  The reference drives every step
// from Python (src/minigpt_infer/engine/engine.py:210-283).
#include <cstring>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "common.h"
#include "launchers.h"

namespace {

// an argument as the recorder stores it: pointers and integers as they are, a float's bits in the low half
typedef unsigned long long Slot;

template <typename T>
T slot_to(Slot v, hipStream_t stream) {
  if constexpr (std::is_same_v<T, hipStream_t>) {
    return stream;  // the recorded stream is the recording's; a replay brings its own
  } else if constexpr (std::is_pointer_v<T>) {
    return reinterpret_cast<T>(v);
  } else if constexpr (std::is_same_v<T, float>) {
    const unsigned int bits = (unsigned int)v;
    float f;
    std::memcpy(&f, &bits, sizeof(f));
    return f;
  } else {
    static_assert(std::is_integral_v<T>, "launcher arguments are pointers, integers and floats");
    return (T)v;
  }
}

template <typename... A, size_t... I>
int invoke(int (*fn)(A...), const Slot* a, hipStream_t stream, std::index_sequence<I...>) {
  return fn(slot_to<A>(a[I], stream)...);
}

struct Launcher {
  const char* name;
  int n_args;
  int (*call)(const Slot*, hipStream_t);
};

template <typename... A>
constexpr int arg_count(int (*)(A...)) { return (int)sizeof...(A); }

template <typename... A>
int call_with(int (*fn)(A...), const Slot* a, hipStream_t stream) {
  return invoke(fn, a, stream, std::index_sequence_for<A...>{});
}

#define MGPT_LAUNCHER_ENTRY(fn) \
  {#fn, arg_count(&fn), [](const Slot* a, hipStream_t s) { return call_with(&fn, a, s); }},
const Launcher kLaunchers[] = {MGPT_FOR_EACH_LAUNCHER(MGPT_LAUNCHER_ENTRY)};
#undef MGPT_LAUNCHER_ENTRY

struct PlannedCall {
  const Launcher* launcher;
  std::vector<Slot> args;
};

struct Plan {
  std::vector<PlannedCall> calls;
};

}  // namespace

extern "C" void* mgpt_plan_create() { return new Plan(); }

extern "C" void mgpt_plan_destroy(void* plan) { delete static_cast<Plan*>(plan); }

extern "C" int mgpt_plan_size(const void* plan) { return plan ? (int)static_cast<const Plan*>(plan)->calls.size() : 0; }

// Appends a call of the launcher `name` with n_args arguments (the stream among them, whatever it
// holds).  MGPT_ERR_BAD_SHAPE for an unknown launcher or a wrong number of arguments.
extern "C" int mgpt_plan_add(void* plan, const char* name, const unsigned long long* args, int n_args) {
  if (!plan || !name || (n_args > 0 && !args)) return MGPT_ERR_NULL;
  for (const Launcher& l : kLaunchers) {
    if (std::strcmp(l.name, name) != 0) continue;
    if (l.n_args != n_args) return MGPT_ERR_BAD_SHAPE;
    static_cast<Plan*>(plan)->calls.push_back({&l, std::vector<Slot>(args, args + n_args)});
    return MGPT_OK;
  }
  return MGPT_ERR_BAD_SHAPE;
}

// Makes the plan's launches on `stream`, in order.  Stops at the first launcher that does not
// return MGPT_OK and returns its code; *failed (if given) is then that call's index.
extern "C" int mgpt_plan_run(const void* plan, hipStream_t stream, int* failed) {
  if (!plan) return MGPT_ERR_NULL;
  const Plan& p = *static_cast<const Plan*>(plan);
  for (size_t i = 0; i < p.calls.size(); ++i) {
    const int rc = p.calls[i].launcher->call(p.calls[i].args.data(), stream);
    if (rc != MGPT_OK) {
      if (failed) *failed = (int)i;
      return rc;
    }
  }
  return MGPT_OK;
}
