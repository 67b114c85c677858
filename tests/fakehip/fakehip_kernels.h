// Argument types of the stand-in runtime's built-in kernels that their callers
// must build themselves.  TEST INFRASTRUCTURE.
#pragma once

// A list of tensors handed to a kernel by value, several KiB long: the shape of
// argument a framework's fused multi-tensor kernels (optimizer steps) take.
struct FakeTensorList {
  float* ptr[300];
  int n[300];
  int count;
  float bias;
};
static_assert(sizeof(FakeTensorList) > 3500 && sizeof(FakeTensorList) <= 4096,
              "a kernel's arguments fit 4 KiB");
