// multi-device-lib-generate: turns a lowered model into the files the runners
// load - the role of the reference's tool of the same name
// (tools/multi-device-lib-generate/multi-device-lib-generate.cpp:41-113,
// lib/Utils/CommandUtils.cpp:85-169).  The reference drives opt -> llc -> c++
// for the host side and opt -> llc (NVPTX) -> ptxas for `ops.ll`; here the
// host side goes through the LLVM tools of the ROCm installation and the
// kernel side becomes a gfx950 code object:
//
//   model.ll  --opt-->  model_opt.ll  --llc-->  model.o  --c++ -shared-->  <out>.so
//   ops.hip   --hipcc --genco-->  <dir of ops>/ops.hsaco           (--device gpu)
//   ops.ll    --clang -target amdgcn-amd-amdhsa-->  .../ops.hsaco  (--device gpu)
//
//   multi-device-lib-generate <model.ll|model.cpp|model.o> [-o <name without extension>]
//       [--device cpu|gpu] [--ops <kernels.hip|kernels.ll>] [--O0|--O1|--O2|--O3]
//       [--saveOptIR] [--saveObject] [--mtriple T] [--mcpu C] [--kcpu gfx950] [--rocm DIR]
//
// The model library is linked against the op and runtime libraries that sit
// beside this tool (../lib), so it loads in any process; the runners would
// also resolve those symbols from their own exports, as the reference's do.
// Exit status 0 on success; the failing command line is printed otherwise.
// Needs no GPU.
#include "multi-device-model-compiler/Runtime/CommandLine.h"

#include <climits>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <sys/stat.h>
#include <sys/wait.h>
#include <unistd.h>
#include <vector>

using namespace multi_device;

static cl::Option Input(cl::Option::Positional, "input", "<input file> model as LLVM IR (.ll), C++ (.cpp) or object (.o)");
static cl::Option Output(cl::Option::String, "o", "Output filename, without extension", "");
static cl::Option Device(cl::Option::String, "device", "Target device: cpu (default) or gpu", "cpu");
static cl::Option Ops(cl::Option::String, "ops", "Kernel source for --device gpu: .hip or AMDGPU LLVM IR (.ll); default <dir of input>/ops.hip", "");
static cl::Option O0(cl::Option::Bool, "O0", "Optimization level 0", "false");
static cl::Option O1(cl::Option::Bool, "O1", "Optimization level 1", "false");
static cl::Option O2(cl::Option::Bool, "O2", "Optimization level 2 (default)", "false");
static cl::Option O3(cl::Option::Bool, "O3", "Optimization level 3", "false");
static cl::Option SaveOptIR(cl::Option::Bool, "saveOptIR", "don't delete opt ir files.", "false");
static cl::Option SaveObject(cl::Option::Bool, "saveObject", "don't delete object files.", "false");
static cl::Option MTriple(cl::Option::String, "mtriple", "Override target triple for module", "");
static cl::Option MCpu(cl::Option::String, "mcpu", "Target cpu", "");
static cl::Option KCpu(cl::Option::String, "kcpu", "Target gpu", "gfx950");
static cl::Option Rocm(cl::Option::String, "rocm", "ROCm installation", "/opt/rocm");

namespace {

bool exists(const std::string &path) {
  struct stat st;
  return ::stat(path.c_str(), &st) == 0;
}

std::string dirOf(const std::string &path) {
  const size_t pos = path.find_last_of('/');
  return pos == std::string::npos ? "." : (pos == 0 ? "/" : path.substr(0, pos));
}

std::string withoutExt(const std::string &path) {
  const size_t dot = path.find_last_of('.');
  const size_t slash = path.find_last_of('/');
  if (dot == std::string::npos || (slash != std::string::npos && dot < slash)) return path;
  return path.substr(0, dot);
}

std::string extOf(const std::string &path) { return path.substr(withoutExt(path).size()); }

// Runs argv[0] with the arguments given and waits for it; prints the command
// line when it fails (lib/Utils/CommandUtils.cpp:48-83 does the same).
int run(const std::vector<std::string> &args) {
  std::vector<char *> argv;
  for (const std::string &a : args) argv.push_back(const_cast<char *>(a.c_str()));
  argv.push_back(nullptr);
  const pid_t pid = ::fork();
  if (pid < 0) {
    std::perror("fork");
    return 1;
  }
  if (pid == 0) {
    ::execvp(argv[0], argv.data());
    std::perror(argv[0]);
    ::_exit(127);
  }
  int status = 0;
  if (::waitpid(pid, &status, 0) < 0) {
    std::perror("waitpid");
    return 1;
  }
  const int rc = WIFEXITED(status) ? WEXITSTATUS(status) : 128 + (WIFSIGNALED(status) ? WTERMSIG(status) : 0);
  if (rc != 0) {
    std::string line;
    for (const std::string &a : args) line += a + " ";
    std::fprintf(stderr, "%s\nProgram path: %s\nCommand execution failed.\n", line.c_str(), args[0].c_str());
  }
  return rc;
}

// Removes a temporary on scope exit unless told to keep it.
struct Remover {
  std::string path;
  bool keep;
  ~Remover() {
    if (!keep && !path.empty()) ::unlink(path.c_str());
  }
};

std::string optLevel() {
  if (O0.asBool()) return "-O0";
  if (O1.asBool()) return "-O1";
  if (O3.asBool()) return "-O3";
  return "-O2";
}

// Directory holding libmgpu_hip_runtime.so and friends: ../lib from this binary.
std::string libDir() {
  char self[PATH_MAX];
  const ssize_t n = ::readlink("/proc/self/exe", self, sizeof(self) - 1);
  if (n <= 0) return "";
  self[n] = '\0';
  const std::string dir = dirOf(dirOf(self)) + "/lib";
  return exists(dir) ? dir : "";
}

int hostLibrary(const std::string &input, const std::string &outputWithExt, bool gpu) {
  const std::string llvmBin = Rocm.str() + "/lib/llvm/bin/";
  const std::string stem = withoutExt(input);
  const std::string ext = extOf(input);
  std::string object = input;
  Remover optRemover{"", SaveOptIR.asBool()}, objRemover{"", SaveObject.asBool()};
  if (ext == ".ll" || ext == ".bc") {
    const std::string optFile = stem + "_opt.ll";
    std::vector<std::string> opt = {llvmBin + "opt", optLevel()};
    if (!MTriple.str().empty()) opt.push_back("-mtriple=" + MTriple.str());
    if (!MCpu.str().empty()) opt.push_back("-mcpu=" + MCpu.str());
    opt.insert(opt.end(), {"-S", "-o", optFile, input});
    if (int rc = run(opt)) {
      std::fprintf(stderr, "Opt LLVM IR wrong.\n");
      return rc;
    }
    optRemover.path = optFile;
    object = stem + ".o";
    std::vector<std::string> llc = {llvmBin + "llc", optLevel()};
    if (!MTriple.str().empty()) llc.push_back("-mtriple=" + MTriple.str());
    if (!MCpu.str().empty()) llc.push_back("-mcpu=" + MCpu.str());
    llc.insert(llc.end(), {"-filetype=obj", "-relocation-model=pic", "-o", object, optFile});
    if (int rc = run(llc)) {
      std::fprintf(stderr, "Gen object file wrong.\n");
      return rc;
    }
    objRemover.path = object;
  } else if (ext == ".cpp" || ext == ".cc") {
    object = stem + ".o";
    std::vector<std::string> cxx = {"c++", optLevel(), "-std=c++17", "-fPIC", "-c", "-o", object, input};
    const std::string lib = libDir();
    if (!lib.empty()) { // the headers of the hand-lowered models sit two levels up from lib/
      cxx.push_back("-I" + dirOf(lib) + "/include");
      cxx.push_back("-I" + dirOf(dirOf(lib)) + "/include");
    }
    if (int rc = run(cxx)) {
      std::fprintf(stderr, "Gen object file wrong.\n");
      return rc;
    }
    objRemover.path = object;
  } else if (ext != ".o") {
    std::fprintf(stderr, "%s: input must be .ll, .bc, .cpp or .o\n", input.c_str());
    return 1;
  }
  std::vector<std::string> link = {"c++", object, "-shared", "-fPIC", "-o", outputWithExt};
  const std::string lib = libDir();
  if (!lib.empty()) {
    link.push_back("-L" + lib);
    if (gpu) {
      link.insert(link.end(), {"-lmgpu_hip_runtime", "-lmgpu_hip_ops"});
    } else {
      link.push_back("-lmcpu_ops");
    }
    link.push_back("-Wl,-rpath," + lib);
  }
  if (int rc = run(link)) {
    std::fprintf(stderr, "Gen library wrong.\n");
    return rc;
  }
  return 0;
}

int kernelModule(const std::string &input) {
  std::string ops = Ops.str();
  if (ops.empty()) {
    ops = dirOf(input) + "/ops.hip";
    if (!exists(ops)) ops = dirOf(input) + "/ops.ll";
  }
  if (!exists(ops)) {
    std::fprintf(stderr, "%s: kernel source not found (give --ops)\n", ops.c_str());
    return 1;
  }
  const std::string out = dirOf(ops) + "/ops.hsaco";
  const std::string ext = extOf(ops);
  std::vector<std::string> cmd;
  if (ext == ".hip") {
    // packed fp32 arithmetic stays off, as everywhere in this library's device code
    cmd = {Rocm.str() + "/bin/hipcc", O0.asBool() ? "-O0" : "-O3", "--offload-arch=" + KCpu.str(), "-Xclang",
           "-target-feature", "-Xclang", "-packed-fp32-ops", "--genco", "-o", out, ops};
  } else if (ext == ".ll" || ext == ".bc") {
    cmd = {Rocm.str() + "/lib/llvm/bin/clang", "-x", "ir", "-target", "amdgcn-amd-amdhsa", "-mcpu=" + KCpu.str(),
           "-nogpulib", O0.asBool() ? "-O0" : "-O3", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-o", out, ops};
  } else {
    std::fprintf(stderr, "%s: kernel source must be .hip, .ll or .bc\n", ops.c_str());
    return 1;
  }
  if (int rc = run(cmd)) {
    std::fprintf(stderr, "Gen code object wrong.\n");
    return rc;
  }
  return 0;
}

} // namespace

int main(int argc, char **argv) {
  if (!cl::ParseCommandLineOptions(argc, argv, "Multi device library generater\n")) {
    std::fprintf(stderr, "Failed to parse options\n");
    return 1;
  }
  const std::string input = Input.str();
  if (!exists(input)) {
    std::fprintf(stderr, "Failed to open input:%s\n", input.c_str());
    return 1;
  }
  std::string output = Output.str();
  const std::string base = output.substr(output.find_last_of("/\\") + 1);
  if (output.empty() || base.find_first_not_of('.') == std::string::npos) {
    if (!output.empty()) std::fprintf(stderr, "Invalid -o option value %s ignored.\n", output.c_str());
    output = withoutExt(input);
  }
  const std::string device = Device.str();
  if (device != "cpu" && device != "gpu" && device != "CPU" && device != "GPU") {
    std::fprintf(stderr, "--device is cpu or gpu\n");
    return 1;
  }
  const bool gpu = device == "gpu" || device == "GPU";
  if (int rc = hostLibrary(input, output + ".so", gpu)) return rc;
  if (gpu) return kernelModule(input);
  return 0;
}
