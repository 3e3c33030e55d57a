// A step as one call: the launches that a step of a given shape makes, recorded
// once as (launcher, arguments) and run again from here, so that the host's
// share of a step that cannot be a HIP graph (prompt portions, whose shapes change
// from step to step) is one call into this library instead of a few hundred calls
// from Python.  Every launcher checks its arguments again when it is run from a
// list, as it does when it is called directly.
#include <cstring>
#include <type_traits>
#include <utility>

#include "api.h"
#include "common.h"

namespace {

// An argument as it lies in a shk_call: pointers and integers as they are, a
// float's bits in the low half.
template <class T>
T as_arg(int64_t v) {
  if constexpr (std::is_pointer_v<T>) {
    return reinterpret_cast<T>(static_cast<intptr_t>(v));
  } else if constexpr (std::is_same_v<T, float>) {
    const uint32_t bits = static_cast<uint32_t>(v);
    float f;
    std::memcpy(&f, &bits, sizeof f);
    return f;
  } else {
    return static_cast<T>(v);
  }
}

// fn(a[0], a[1], ..., stream): every launcher's last parameter is its stream.
template <class... Args, size_t... I>
int invoke(int (*fn)(Args...), const int64_t* a, void* stream, std::index_sequence<I...>) {
  constexpr size_t last = sizeof...(Args) - 1;
  return fn((I == last ? as_arg<Args>(static_cast<int64_t>(reinterpret_cast<intptr_t>(stream)))
                       : as_arg<Args>(a[I]))...);
}

template <class... Args>
int call(int (*fn)(Args...), const int64_t* a, void* stream) {
  static_assert(sizeof...(Args) >= 1 && sizeof...(Args) <= SHK_CALL_MAX_ARGS, "too many arguments for a shk_call");
  return invoke(fn, a, stream, std::index_sequence_for<Args...>{});
}

struct Launcher {
  const char* name;
  int (*run)(const int64_t* a, void* stream);
};

#define SHK_LAUNCHER(f) \
  { #f, [](const int64_t* a, void* stream) { return call(f, a, stream); } }

// the launchers of api.h that take a stream (the queries and the one-time re-layouts of
// weights are not steps' business)
const Launcher kLaunchers[] = {
    SHK_LAUNCHER(shk_copy_words),
    SHK_LAUNCHER(shk_gather_rows),
    SHK_LAUNCHER(shk_zero_bytes),
    SHK_LAUNCHER(shk_embed),
    SHK_LAUNCHER(shk_add_rmsnorm),
    SHK_LAUNCHER(shk_act_mul),
    SHK_LAUNCHER(shk_gemm),
    SHK_LAUNCHER(shk_gemm_bf16_tiled_weight),
    SHK_LAUNCHER(shk_rope_kv_store),
    SHK_LAUNCHER(shk_attention),
    SHK_LAUNCHER(shk_attention_decode_bf16),
    SHK_LAUNCHER(shk_attention_prefill_bf16),
    SHK_LAUNCHER(shk_attention_prefill_shared_bf16),
    SHK_LAUNCHER(shk_argmax),
    SHK_LAUNCHER(shk_sample),
};
constexpr int kNumLaunchers = sizeof(kLaunchers) / sizeof(kLaunchers[0]);

}  // namespace

extern "C" int shk_call_id(const char* name) {
  if (!name) return -1;
  for (int i = 0; i < kNumLaunchers; ++i)
    if (std::strcmp(kLaunchers[i].name, name) == 0) return i;
  return -1;
}

extern "C" int shk_run_calls(const shk_call* calls, int n, void* stream) {
  SHK_REQUIRE(n >= 0 && (calls || n == 0), "run_calls: bad list");
  for (int i = 0; i < n; ++i) {
    const int id = calls[i].launcher;
    SHK_REQUIRE(id >= 0 && id < kNumLaunchers, "run_calls: call %d names launcher %d, which does not exist", i, id);
    const int status = kLaunchers[id].run(calls[i].args, stream);
    if (status != 0) return status;  // the launcher's message stands; calls before it have run
  }
  return 0;
}
