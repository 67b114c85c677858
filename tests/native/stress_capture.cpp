// Host-only stress of the interception layer and the scheduler, meant to be
// built with -fsanitize=thread together with the library sources: client
// threads push records through the lock-free hand-off while the scheduler
// thread runs the three-phase schedule, against the recording HIP stand-in.
// TEST INFRASTRUCTURE.  Exit status 0 = outputs equal the isolated result and
// (under ThreadSanitizer) no data race was reported.
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <atomic>
#include <string>
#include <thread>
#include <vector>

#include "orion_scheduler.h"

extern "C" void fake_kernel_saxpy(void** p);
extern "C" void fake_kernel_sqadd(void** p);
extern "C" void fakehip_set_costs(long long kernel_ns, long long copy_ns);

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

void expected(int c, int iters, float* y) {
  float x[kN];
  for (int i = 0; i < kN; ++i) { x[i] = (float)i / kN + c; y[i] = 0.0f; }
  for (int it = 0; it < iters; ++it)
    for (int k = 0; k < g_kernels[(size_t)c]; ++k)
      for (int i = 0; i < kN; ++i)
        y[i] = (k % 2 == 0) ? 0.5f * x[i] + y[i] : y[i] * y[i] + 0.125f;
}

void client(int c) {
  g_tids[(size_t)c] = (int)syscall(SYS_gettid);
  g_tids_ready.fetch_add(1);
  float host_x[kN];
  for (int i = 0; i < kN; ++i) host_x[i] = (float)i / kN + c;
  pthread_barrier_wait(&g_barrier);   // released once setup() has run
  float *y = nullptr, *x = nullptr;
  if (hipMalloc((void**)&y, kN * 4) != hipSuccess || hipMalloc((void**)&x, kN * 4) != hipSuccess) exit(3);
  float zeros[kN] = {0};
  hipMemcpy(y, zeros, kN * 4, hipMemcpyHostToDevice);
  int n = kN;
  float a = 0.5f, cc = 0.125f;
  int it = 0;
  while (it < g_iters[(size_t)c]) {
    hipMemcpyAsync(x, host_x, kN * 4, hipMemcpyHostToDevice, nullptr);
    for (int k = 0; k < g_kernels[(size_t)c]; ++k) {
      if (k % 2 == 0) {
        void* params[] = {&y, &x, &a, &n};
        if (hipModuleLaunchKernel((hipFunction_t)fake_kernel_saxpy, 1, 1, 1, 64, 1, 1, 0, nullptr, params, nullptr) != hipSuccess) exit(4);
      } else {
        void* params[] = {&y, &cc, &n};
        if (hipModuleLaunchKernel((hipFunction_t)fake_kernel_sqadd, 1, 1, 1, 64, 1, 1, 0, nullptr, params, nullptr) != hipSuccess) exit(4);
      }
    }
    block(it);
    ++it;
    g_done[(size_t)c] = it;
    if (it == 1 || it == 10) pthread_barrier_wait(&g_barrier);
    if (stop()) break;
  }
  pthread_barrier_wait(&g_barrier);
  g_out[(size_t)c].resize(kN);
  hipMemcpy(g_out[(size_t)c].data(), y, kN * 4, hipMemcpyDeviceToHost);
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
  std::vector<std::string> files;
  for (int c = 0; c < g_clients; ++c) {
    g_kernels[(size_t)c] = 5 + c;
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
  if (g_done.back() != hp_iters) bad = 1;
  return bad;
}
