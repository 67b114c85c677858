// The name a kernel goes by in a profile CSV and in the scheduler's reports:
// the runtime's (mangled) name, demangled, without template and call arguments
// and without characters the CSV's parser splits on
// (reference: the Name column of profiling/postprocessing/generate_file.py:176-179,
// which a ',' would break in populate_kernel_info, scheduler_eval.cpp:514-520).
#pragma once

#include <cxxabi.h>
#include <stdlib.h>
#include <string.h>

#include <string>

namespace orion {

inline std::string short_kernel_name(const char* mangled) {
  if (!mangled || !*mangled) return "unknown";
  int status = 0;
  char* dem = abi::__cxa_demangle(mangled, nullptr, nullptr, &status);
  std::string s = (status == 0 && dem) ? dem : mangled;
  free(dem);
  for (size_t at; (at = s.find("(anonymous namespace)::")) != std::string::npos;)
    s.erase(at, strlen("(anonymous namespace)::"));
  size_t cut = s.find_first_of("<(");
  if (cut != std::string::npos && cut > 0) s = s.substr(0, cut);
  for (char& c : s)
    if (c == ',' || c == '\n') c = ';';
  return s;
}

}  // namespace orion
