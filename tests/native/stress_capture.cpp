// Host-only stress of the interception layer and the scheduler, meant to be
// built with -fsanitize=thread together with the library sources: client
// threads push records through the lock-free hand-off while the scheduler
// thread runs the three-phase schedule, against the recording HIP stand-in.
// TEST INFRASTRUCTURE.  Exit status 0 = outputs equal the isolated result and
// (under ThreadSanitizer) no data race was reported.
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <dlfcn.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <atomic>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "orion_scheduler.h"
#include "../fakehip/fakehip_kernels.h"

extern "C" void fake_kernel_saxpy(void** p);
extern "C" void fake_kernel_sqadd(void** p);
extern "C" void fake_kernel_multi(void** p);
extern "C" void fakehip_set_costs(long long kernel_ns, long long copy_ns);
extern "C" long fakehip_repointed_nodes(void);
extern "C" void orion_register_stream(void* stream);
extern "C" void orion_tls_fresh_stats(unsigned long long* reloads, unsigned long long* touches);

namespace {

constexpr int kN = 64;
int g_clients = 3;
std::vector<int> g_kernels;   // per client, per iteration
std::vector<int> g_iters;     // iteration limit
std::vector<int> g_done;      // iterations completed
std::vector<int> g_tids;
std::vector<std::vector<float>> g_out;
pthread_barrier_t g_barrier;  // clients + scheduler
std::atomic<int> g_tids_ready{0};

// A caching allocator in miniature: a client hands a temporary back to its pool
// as soon as the last kernel using it has been *launched* (safe in stream order)
// and takes it from there again; a thread that is no client of the scheduler
// returns the pools' blocks to the runtime now and then, holding the pool lock
// while it does -- what a framework's allocator does when it trims its cache.
// hipFree must not release a block that a queued record still names.
std::mutex g_pool_lock;
std::vector<std::vector<float*>> g_pool;
std::atomic<bool> g_trim_stop{false};
std::atomic<long> g_trimmed{0};

float* pool_get(int c) {
  // the runtime is asked for memory with the pool lock held, as a caching
  // allocator does: the call must not wait for anything another client's
  // progress decides
  std::lock_guard<std::mutex> hold(g_pool_lock);
  auto& mine = g_pool[(size_t)c];
  if (!mine.empty()) { float* t = mine.back(); mine.pop_back(); return t; }
  float* t = nullptr;
  if (hipMalloc((void**)&t, kN * 4) != hipSuccess) exit(3);
  return t;
}

void pool_put(int c, float* t) {
  std::lock_guard<std::mutex> hold(g_pool_lock);
  g_pool[(size_t)c].push_back(t);
}

void trimmer() {
  // STRESS_DLOPEN names a small library that this thread keeps loading and
  // unloading, as a framework loads code lazily: every change in the set of loaded
  // libraries makes the interception library reload its thread-local helper while
  // client threads are calling into it
  const char* churn = getenv("STRESS_DLOPEN");
  while (!g_trim_stop.load()) {
    if (churn && *churn) {
      if (void* h = dlopen(churn, RTLD_NOW | RTLD_LOCAL)) dlclose(h);
    }
    {
      std::lock_guard<std::mutex> hold(g_pool_lock);
      for (auto& pool : g_pool) {
        for (float* t : pool) { if (hipFree(t) != hipSuccess) exit(6); g_trimmed.fetch_add(1); }
        pool.clear();
      }
    }
    usleep(50);
  }
}

// Kernel k of an iteration: every fifth one scales the output through a list of
// tensors passed by value; of the others, even ones add x, odd ones square.
inline bool is_multi(int k) { return k % 5 == 4; }
inline float step_of(int k, float x, float y) {
  if (is_multi(k)) return y * 0.75f + 0.0625f;
  return (k % 2 == 0) ? 0.5f * x + y : y * y + 0.125f;
}

// The list-of-tensors kernel through each launch form; the list lives on this
// function's stack and is overwritten before it returns.
struct ClientState;
hipError_t launch_multi(ClientState& st, int form);

void expected(int c, int iters, float* y) {
  float x[kN];
  for (int i = 0; i < kN; ++i) { x[i] = (float)i / kN + c; y[i] = 0.0f; }
  for (int it = 0; it < iters; ++it)
    for (int k = 0; k < g_kernels[(size_t)c]; ++k)
      for (int i = 0; i < kN; ++i)
        y[i] = step_of(k, x[i], y[i]);
}

// What a client is made of: its buffers, the stream its calls name, and what its
// output must be by now.
struct ClientState {
  int c;
  float *y = nullptr, *x = nullptr;
  hipStream_t stream = nullptr;
  float want[kN];
  float host_x[kN];
};

// One kernel of client `st.c`'s iteration `it`, through one of the launch forms a
// framework's libraries use, on the stream the client names.  Callable from any
// thread: calls that name the client's stream are the client's.
void launch_one(ClientState& st, int k, int it) {
  const int c = st.c;
  if (is_multi(k)) {
    if (launch_multi(st, (k + it) % 3) != hipSuccess) exit(4);
    if (hipGetLastError() != hipSuccess) { fprintf(stderr, "client %d: stale error after a launch\n", c); exit(7); }
    for (int i = 0; i < kN; ++i) st.want[i] = step_of(k, st.host_x[i], st.want[i]);
    return;
  }
  int n = kN;
  float a = 0.5f, cc = 0.125f;
  // even kernels read x through a pooled temporary: cleared by a fill, then
  // written by a device copy (both are records that can be queued ahead)
  float* temp = nullptr;
  if (k % 2 == 0) {
    temp = pool_get(c);
    if (hipMemsetAsync(temp, 0, kN * 4, st.stream) != hipSuccess) exit(4);
    if (hipMemcpyAsync(temp, st.x, kN * 4, hipMemcpyDeviceToDevice, st.stream) != hipSuccess) exit(4);
  }
  // private copies of the arguments, overwritten as soon as the call has
  // returned: a queued record must own what it needs
  float* my_y = st.y; float* my_x = temp ? temp : st.x; float my_a = a, my_c = cc; int my_n = n;
  void* saxpy_params[] = {&my_y, &my_x, &my_a, &my_n};
  void* sqadd_params[] = {&my_y, &my_c, &my_n};
  void* fn = k % 2 == 0 ? (void*)fake_kernel_saxpy : (void*)fake_kernel_sqadd;
  void** params = k % 2 == 0 ? saxpy_params : sqadd_params;
  hipError_t rc;
  switch ((k + it) % 3) {
    case 0:   // module launch with a kernelParams array
      rc = hipModuleLaunchKernel((hipFunction_t)fn, 1, 1, 1, 64, 1, 1, 0, st.stream, params, nullptr);
      break;
    case 1:   // argument sizes known to the runtime only
      // the two kernels have different launch bounds and are launched with
      // blocks of that size, like a framework's kernels
      rc = hipLaunchKernel(fn, dim3(1), dim3(k % 2 == 0 ? 256 : 64), params, 0, st.stream);
      break;
    default: {  // module launch with one argument buffer
      struct { float* y; float* x; float a; int n; } saxpy_buf = {my_y, my_x, my_a, my_n};
      struct { float* y; float c; int n; } sqadd_buf = {my_y, my_c, my_n};
      void* buf = k % 2 == 0 ? (void*)&saxpy_buf : (void*)&sqadd_buf;
      size_t size = k % 2 == 0 ? sizeof saxpy_buf : sizeof sqadd_buf;
      void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, buf, HIP_LAUNCH_PARAM_BUFFER_SIZE,
                       &size, HIP_LAUNCH_PARAM_END};
      rc = hipModuleLaunchKernel((hipFunction_t)fn, 1, 1, 1, 64, 1, 1, 0, st.stream, nullptr, extra);
      memset(&saxpy_buf, 0xff, sizeof saxpy_buf);
      memset(&sqadd_buf, 0xff, sizeof sqadd_buf);
      size = 0;
    }
  }
  if (rc != hipSuccess) exit(4);
  // a framework's launch check: whatever the library did on this thread to
  // queue the call, it must not leave an error of its own behind
  if (hipGetLastError() != hipSuccess) { fprintf(stderr, "client %d: stale error after a launch\n", c); exit(7); }
  if (temp) pool_put(c, temp);
  my_y = my_x = nullptr; my_a = my_c = -1e30f; my_n = -1;
  for (int i = 0; i < kN; ++i) st.want[i] = step_of(k, st.host_x[i], st.want[i]);
}

hipError_t launch_multi(ClientState& st, int form) {
  // the output as four tensors of a long list; the unused entries are poison
  FakeTensorList list;
  memset(&list, 0x5a, sizeof list);
  list.count = 4;
  list.bias = 0.0625f;
  for (int t = 0; t < 4; ++t) { list.ptr[t] = st.y + t * (kN / 4); list.n[t] = kN / 4; }
  float scale = 0.75f;
  void* params[] = {&list, &scale};
  hipError_t rc;
  if (form == 0) {
    rc = hipModuleLaunchKernel((hipFunction_t)fake_kernel_multi, 1, 1, 1, 64, 1, 1, 0, st.stream,
                               params, nullptr);
  } else if (form == 1) {
    rc = hipLaunchKernel((void*)fake_kernel_multi, dim3(1), dim3(512), params, 0, st.stream);
  } else {
    struct { FakeTensorList list; float scale; } buf;
    memcpy(&buf.list, &list, sizeof list);
    buf.scale = scale;
    size_t size = sizeof buf;
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &buf, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                     HIP_LAUNCH_PARAM_END};
    rc = hipModuleLaunchKernel((hipFunction_t)fake_kernel_multi, 1, 1, 1, 64, 1, 1, 0, st.stream,
                               nullptr, extra);
    memset(&buf, 0xff, sizeof buf);
    size = 0;
  }
  memset(&list, 0xff, sizeof list);
  scale = -1e30f;
  return rc;
}

// A thread that is no client of the scheduler and launches the second half of
// every training client's iteration for it, on that client's stream, while the
// client waits -- what a framework's one autograd thread per device does for all
// the trainers of a process.
struct WorkerTask { ClientState* st; int first, last, it; std::atomic<int>* done; };
std::mutex g_worker_lock;
std::vector<WorkerTask> g_worker_tasks;
std::atomic<bool> g_worker_stop{false};

void worker() {
  while (!g_worker_stop.load()) {
    WorkerTask task;
    {
      std::lock_guard<std::mutex> hold(g_worker_lock);
      if (g_worker_tasks.empty()) { task.st = nullptr; }
      else { task = g_worker_tasks.front(); g_worker_tasks.erase(g_worker_tasks.begin()); }
    }
    if (!task.st) { usleep(20); continue; }
    for (int k = task.first; k < task.last; ++k) launch_one(*task.st, k, task.it);
    task.done->store(1, std::memory_order_release);
  }
}

// Reads the client's output back in the middle of the run and compares it with
// what the kernels launched so far must have produced: a wait or a copy that
// overtakes queued work, or work that ran out of order, shows here.
void check_now(ClientState& st, int it, hipEvent_t ev) {
  float got[kN];
  if (it % 2 == 0) {
    // an event recorded behind the work, waited for on the host, then an
    // asynchronous copy and a stream wait
    if (hipEventRecord(ev, st.stream) != hipSuccess || hipEventSynchronize(ev) != hipSuccess) exit(8);
    if (hipMemcpyAsync(got, st.y, kN * 4, hipMemcpyDeviceToHost, st.stream) != hipSuccess) exit(8);
    if (hipStreamSynchronize(st.stream) != hipSuccess) exit(8);
  } else {
    if (hipMemcpy(got, st.y, kN * 4, hipMemcpyDeviceToHost) != hipSuccess) exit(8);   // blocking
  }
  if (memcmp(got, st.want, sizeof got) != 0) {
    fprintf(stderr, "client %d: output read back in iteration %d differs from what its kernels "
                    "must have produced by then\n", st.c, it);
    exit(9);
  }
}

void client(int c) {
  g_tids[(size_t)c] = (int)syscall(SYS_gettid);
  g_tids_ready.fetch_add(1);
  static ClientState states[64];
  ClientState& st = states[c];
  st.c = c;
  for (int i = 0; i < kN; ++i) { st.host_x[i] = (float)i / kN + c; st.want[i] = 0.0f; }
  pthread_barrier_wait(&g_barrier);   // released once setup() has run
  // a stream of the client's own, as a framework client has: calls that name it
  // are this client's, whichever thread makes them
  if (hipStreamCreateWithFlags(&st.stream, hipStreamNonBlocking) != hipSuccess) exit(3);
  orion_register_stream(st.stream);
  hipEvent_t ev;
  if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) exit(3);
  if (hipMalloc((void**)&st.y, kN * 4) != hipSuccess || hipMalloc((void**)&st.x, kN * 4) != hipSuccess) exit(3);
  float zeros[kN] = {0};
  hipMemcpy(st.y, zeros, kN * 4, hipMemcpyHostToDevice);
  const bool trains = c != g_clients - 1;
  const int nk = g_kernels[(size_t)c];
  int it = 0;
  while (it < g_iters[(size_t)c]) {
    hipMemcpyAsync(st.x, st.host_x, kN * 4, hipMemcpyHostToDevice, st.stream);
    const int half = trains ? nk / 2 : nk;
    for (int k = 0; k < half; ++k) launch_one(st, k, it);
    if (half < nk) {
      std::atomic<int> done{0};
      {
        std::lock_guard<std::mutex> hold(g_worker_lock);
        g_worker_tasks.push_back({&st, half, nk, it, &done});
      }
      // Meanwhile this thread makes blocking calls of its own: two threads of
      // one client in the queue at once, one waiting for each of its records,
      // the other (when records are queued ahead) racing up to a whole ring
      // ahead of it.  Each blocking call must be carried out and must hand back
      // its own result: x does not change during an iteration.
      long reads = 0;
      while (!done.load(std::memory_order_acquire)) {
        float got[kN];
        memset(got, 0xee, sizeof got);
        if (hipMemcpy(got, st.x, kN * 4, hipMemcpyDeviceToHost) != hipSuccess) exit(10);
        if (memcmp(got, st.host_x, sizeof got) != 0) {
          fprintf(stderr, "client %d: a blocking copy made while another thread of the client "
                          "launches was not carried out (iteration %d, read %ld)\n", c, it, reads);
          exit(11);
        }
        float* scratch = nullptr;
        if (hipMalloc((void**)&scratch, 256) != hipSuccess || scratch == nullptr) exit(12);
        if (hipFree(scratch) != hipSuccess) exit(12);
        ++reads;
      }
    }
    if (it % 3 == 2) check_now(st, it, ev);
    block(it);
    ++it;
    g_done[(size_t)c] = it;
    if (it == 1 || it == 10) pthread_barrier_wait(&g_barrier);
    if (stop()) break;
  }
  pthread_barrier_wait(&g_barrier);
  g_out[(size_t)c].resize(kN);
  hipMemcpy(g_out[(size_t)c].data(), st.y, kN * 4, hipMemcpyDeviceToHost);
}

}  // namespace

int main(int argc, char** argv) {
  const char* dir = argc > 1 ? argv[1] : "/tmp";
  if (argc > 2) g_clients = atoi(argv[2]);
  const int hp_iters = argc > 3 ? atoi(argv[3]) : 60;
  fakehip_set_costs(20000, 3000);
  g_kernels.resize((size_t)g_clients);
  g_iters.assign((size_t)g_clients, 1000000);
  g_iters.back() = hp_iters;
  g_done.assign((size_t)g_clients, 0);
  g_tids.assign((size_t)g_clients, 0);
  g_out.resize((size_t)g_clients);
  g_pool.resize((size_t)g_clients);
  std::vector<std::string> files;
  for (int c = 0; c < g_clients; ++c) {
    // the first best-effort client's iterations are longer than its queue: when
    // the job ends, its queue is full of records nobody waits for
    g_kernels[(size_t)c] = (c == 0 && g_clients > 2) ? 150 : 5 + c;
    files.push_back(std::string(dir) + "/stress_client" + std::to_string(c) + ".csv");
    FILE* f = fopen(files.back().c_str(), "w");
    if (!f) return 5;
    fprintf(f, "Name,Profile,Memory_footprint,SM_usage,Duration\n");
    for (int k = 0; k < g_kernels[(size_t)c]; ++k)
      fprintf(f, "k%d,%d,0,%d,%d\n", k, (k + c) % 3 - 1, 20 + 37 * k, 8000 + 5000 * k);
    fclose(f);
  }
  pthread_barrier_init(&g_barrier, nullptr, (unsigned)g_clients + 1);
  std::vector<std::thread> threads;
  for (int c = 0; c < g_clients; ++c) threads.emplace_back(client, c);
  while (g_tids_ready.load() < g_clients) usleep(100);

  std::vector<char*> names, paths;
  std::vector<int> nk = g_kernels, ni = g_iters;
  std::vector<unsigned char> train((size_t)g_clients, 1);
  train.back() = 0;
  for (auto& f : files) { names.push_back((char*)"stress"); paths.push_back((char*)f.c_str()); }
  std::thread trim_thread(trimmer);
  std::thread worker_thread(worker);
  void* s = sched_init();
  setup(s, g_clients, g_tids.data(), names.data(), paths.data(), nk.data(), ni.data(),
        (bool*)train.data(), false);
  pthread_barrier_wait(&g_barrier);
  schedule(s, g_clients, true, 0, true, 1, false, false, 100000, 1, 1);
  pthread_barrier_wait(&g_barrier);
  schedule(s, g_clients, true, 0, true, 10, false, false, 100000, 1, 1);
  pthread_barrier_wait(&g_barrier);
  schedule(s, g_clients, true, 0, false, 0, false, false, 100000, 1, 1);
  pthread_barrier_wait(&g_barrier);
  for (auto& t : threads) t.join();
  g_trim_stop.store(true);
  trim_thread.join();
  g_worker_stop.store(true);
  worker_thread.join();
  orion_sched_teardown();

  int bad = 0;
  for (int c = 0; c < g_clients; ++c) {
    float want[kN];
    expected(c, g_done[(size_t)c], want);
    if (memcmp(want, g_out[(size_t)c].data(), sizeof want) != 0) {
      fprintf(stderr, "client %d: output differs after %d iterations\n", c, g_done[(size_t)c]);
      bad = 1;
    }
    printf("client %d: %d iterations\n", c, g_done[(size_t)c]);
  }
  printf("%ld pooled blocks returned to the runtime while the clients ran\n", g_trimmed.load());
  if (g_trimmed.load() == 0) bad = 1;
  // no graph kernel node may ever be given the parameters of another kernel
  // than the one it was created for
  printf("%ld graph kernel nodes re-pointed to another kernel\n", fakehip_repointed_nodes());
  if (fakehip_repointed_nodes() != 0) bad = 1;
  if (g_done.back() != hp_iters) bad = 1;
  if (const char* want = getenv("STRESS_EXPECT_TLS_RELOADS")) {
    unsigned long long reloads = 0, touches = 0;
    orion_tls_fresh_stats(&reloads, &touches);
    printf("thread-local helper: %llu reloads, %llu calls into a fresh copy\n", reloads, touches);
    if (reloads < (unsigned long long)atoll(want) || touches < reloads) bad = 1;
  }
  return bad;
}
