// Keeps the thread-local accesses of client threads on the dynamic loader's
// fast path.
//
// Code in a shared library reaches its thread-local variables through
// __tls_get_addr, which compares the calling thread's table of thread-local
// blocks (its "generation") with the loader's global one.  On glibc before 2.39
// (bug 19924) a thread only ever catches up to the generation of the newest
// library whose thread-local storage it touches: once any library with
// thread-local storage has been loaded -- or any such library unloaded -- after
// that one, every thread-local access the thread makes through __tls_get_addr
// takes the slow path, for the rest of the thread's life.  A framework client
// makes dozens of such accesses per operator (dispatch keys, autograd and
// allocator state), and a process that loads libraries lazily (solver
// libraries, code-object loaders) is in that state from its first request on:
// the ResNet-50 bs4 request measured 0.25 ms (7 %) longer to submit, with or
// without this library in the process.
//
// The cure is to let the thread touch thread-local storage of a library that is
// newer than everything else: liborion_tlsfresh.so is (re)loaded whenever the
// process's set of loaded libraries has changed, and every client thread calls
// into it once after each reload.  This library's own thread-local variables use
// the initial-exec model and never go through __tls_get_addr.
//
// ORION_TLS_REFRESH=0 switches all of it off.
#pragma once

#include <atomic>
#include <cstdint>

namespace orion {

extern std::atomic<uint32_t> g_tls_fresh_reloads;   // bumped after every reload
extern __thread uint32_t tl_tls_fresh_seen __attribute__((tls_model("initial-exec")));

void tls_fresh_touch_slow();

// Once per reload and thread: call into the freshly loaded library.  Cheap
// enough for every intercepted call (one relaxed load and a compare).
inline void tls_fresh_touch() {
  if (tl_tls_fresh_seen != g_tls_fresh_reloads.load(std::memory_order_relaxed))
    tls_fresh_touch_slow();
}

// Reloads the library if the process has loaded or unloaded anything since the
// last reload, then touches.  For the places a thread passes once per iteration
// (block, stop, the scheduler's end of an iteration).
void tls_fresh_check();

}  // namespace orion
