// Plan-driven models for the runners (see Runtime/PlanModel.h).
#include "multi-device-model-compiler/Runtime/PlanModel.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

namespace multi_device {

using namespace conversion;

bool IsPlanFile(const std::string &path) {
  return path.size() > 5 && path.compare(path.size() - 5, 5, ".plan") == 0;
}

PlanModel *PlanModel::Load(const std::string &path, DeviceType device) {
  std::ifstream in(path);
  if (!in) {
    std::fprintf(stderr, "Failed to open plan:%s\n", path.c_str());
    return nullptr;
  }
  std::stringstream text;
  text << in.rdbuf();
  PlanModel *m = new PlanModel();
  std::string error;
  if (!parseDevicePlan(text.str(), m->plan, error) || !verifyDevicePlan(m->plan, error) ||
      !lowerToRuntimeCalls(m->plan, device, m->program, error) || !checkRuntimeProgram(m->program, error)) {
    std::fprintf(stderr, "%s: %s\n", path.c_str(), error.c_str());
    delete m;
    return nullptr;
  }
  const size_t slash = path.find_last_of('/');
  const std::string dir = slash == std::string::npos ? std::string() : path.substr(0, slash);
  if (!loadPlanConstants(m->plan, dir, m->buffers, error)) {
    std::fprintf(stderr, "%s\n", error.c_str());
    delete m;
    return nullptr;
  }
  return m;
}

PlanModel::~PlanModel() {
  for (void *p : buffers) std::free(p);
}

bool PlanModel::PrepareIO(const std::vector<std::string> &files) {
  if (!files.empty() && files.size() != plan.inputs.size()) {
    std::fprintf(stderr, "Data num not equal input num!");
    return false;
  }
  for (size_t i = 0; i < plan.inputs.size(); i++) {
    const int v = plan.inputs[i];
    const size_t bytes = plan.values[v].type.bytes();
    std::free(buffers[v]);
    buffers[v] = std::calloc(bytes ? bytes : 1, 1);
    if (files.empty()) continue;
    FILE *f = std::fopen(files[i].c_str(), "rb");
    if (!f) {
      std::fprintf(stderr, "Failed to open file:%s\n", files[i].c_str());
      return false;
    }
    std::fseek(f, 0, SEEK_END);
    const long size = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    const bool ok = (size_t)size == bytes && std::fread(buffers[v], 1, bytes, f) == bytes;
    std::fclose(f);
    if (!ok) {
      std::fprintf(stderr, "Wrong File size\n");
      return false;
    }
  }
  for (int v : plan.outputs) {
    const size_t bytes = plan.values[v].type.bytes();
    std::free(buffers[v]);
    buffers[v] = std::calloc(bytes ? bytes : 1, 1);
  }
  return true;
}

bool PlanModel::Run(void *library) {
  std::string error;
  if (!executeRuntimeProgram(plan, program, buffers, library, error)) {
    std::fprintf(stderr, "%s\n", error.c_str());
    return false;
  }
  return true;
}

bool PlanModel::SaveOutput(size_t idx, const std::string &file) const {
  if (idx >= plan.outputs.size()) return false;
  const int v = plan.outputs[idx];
  FILE *f = std::fopen(file.c_str(), "wb");
  if (!f) {
    std::fprintf(stderr, "Failed to open file:%s\n", file.c_str());
    return false;
  }
  const size_t bytes = plan.values[v].type.bytes();
  const bool ok = std::fwrite(buffers[v], 1, bytes, f) == bytes;
  std::fclose(f);
  return ok;
}

} // namespace multi_device
