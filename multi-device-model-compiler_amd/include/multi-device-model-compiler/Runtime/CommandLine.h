// Minimal command-line registry standing in for llvm::cl, which the reference
// runners use (tools/multi-device-gpu-runner/multi-device-gpu-runner.cpp:16-41,
// lib/Runtime/ModelInfo.cpp:10-28).  Same surface: named options taking a value
// (`--name value`, `--name=value`, one or two leading dashes), boolean flags,
// comma separated lists that may repeat, one required positional argument.
#ifndef MULTI_DEVICE_MODEL_COMPILER_RUNTIME_COMMANDLINE_H_
#define MULTI_DEVICE_MODEL_COMPILER_RUNTIME_COMMANDLINE_H_

#include <string>
#include <vector>

namespace multi_device {
namespace cl {

struct Option {
  enum Kind { String, Int, Bool, List, Positional };
  Option(Kind kind, const char *name, const char *desc, const char *init = "");
  Kind kind;
  std::string name, desc, value;
  std::vector<std::string> values; // List
  std::string initial_;
  bool seen = false;

  const std::string &str() const { return value; }
  int asInt() const;
  bool asBool() const;
};

// Parses argv against every Option constructed so far.  Returns false (after
// printing to stderr) on an unknown option, a missing value or a missing
// positional argument; `--help` prints the option table and exits 0.
bool ParseCommandLineOptions(int argc, char **argv, const char *overview);

// Clears parsed state (tests parse several command lines in one process).
void ResetAllOptions();

} // namespace cl
} // namespace multi_device

#endif
