#include "multi-device-model-compiler/Runtime/RuntimeUtil.h"

#include <cerrno>
#include <cstdio>
#include <cstring>
#include <dlfcn.h>

namespace multi_device {

void *LoadRawData(const std::string &file, size_t numElements, size_t elementBytes) {
  std::FILE *f = std::fopen(file.c_str(), "rb");
  if (!f) {
    std::fprintf(stderr, "Error reading file: %s\n", std::strerror(errno));
    return nullptr;
  }
  std::fseek(f, 0, SEEK_END);
  const long fileSize = std::ftell(f);
  std::fseek(f, 0, SEEK_SET);
  const size_t want = numElements * elementBytes;
  if (fileSize < 0 || (size_t)fileSize < want) {
    std::fprintf(stderr, "Wrong File size\n");
    std::fclose(f);
    return nullptr;
  }
  void *data = std::aligned_alloc(64, (want + 63) / 64 * 64 + 64);
  const size_t got = std::fread(data, 1, want, f);
  std::fclose(f);
  if (got != want) {
    std::fprintf(stderr, "Error reading file: short read\n");
    std::free(data);
    return nullptr;
  }
  return data;
}

float *LoadFloatData(std::string &file, size_t numElements) {
  return static_cast<float *>(LoadRawData(file, numElements, sizeof(float)));
}

static bool saveRaw(const std::string &file, const void *data, size_t bytes) {
  std::FILE *f = std::fopen(file.c_str(), "wb");
  if (!f) {
    std::fprintf(stderr, "Error open file to write:%s\n", std::strerror(errno));
    return false;
  }
  const size_t put = data ? std::fwrite(data, 1, bytes, f) : 0;
  std::fclose(f);
  return put == bytes;
}

template <size_t N> void SaveFloatData(std::string &file, FloatTensor<N> *tensor) {
  saveRaw(file, tensor->aligned, tensor->GetNumElements() * sizeof(float));
}
template void SaveFloatData<1>(std::string &, FloatTensor<1> *);
template void SaveFloatData<2>(std::string &, FloatTensor<2> *);
template void SaveFloatData<3>(std::string &, FloatTensor<3> *);
template void SaveFloatData<4>(std::string &, FloatTensor<4> *);
template void SaveFloatData<5>(std::string &, FloatTensor<5> *);

namespace {
// The descriptor layout does not depend on the element type; only the byte
// size of the buffer does.
template <size_t N>
FloatTensor<N> *initTensorDescripter(std::vector<size_t> &shapes, const std::string &file, bool init,
                                     bool useFile, size_t elementBytes) {
  FloatTensor<N> *tensor = FloatTensor<N>::CreateTensor(shapes);
  if (init) {
    const size_t num = tensor->GetNumElements();
    void *data = useFile ? LoadRawData(file, num, elementBytes)
                         : std::aligned_alloc(64, (num * elementBytes + 63) / 64 * 64 + 64);
    tensor->InitData(static_cast<float *>(data));
  }
  return tensor;
}

template <typename F> bool withRank(size_t rank, F &&f) {
  switch (rank) {
  case 1:
    f(std::integral_constant<size_t, 1>());
    return true;
  case 2:
    f(std::integral_constant<size_t, 2>());
    return true;
  case 3:
    f(std::integral_constant<size_t, 3>());
    return true;
  case 4:
    f(std::integral_constant<size_t, 4>());
    return true;
  case 5:
    f(std::integral_constant<size_t, 5>());
    return true;
  default:
    return false;
  }
}
} // namespace

void *GetTensorDescripter(std::vector<size_t> &shapes, std::string file, bool init, bool useFile,
                          size_t elementBytes) {
  void *tensor = nullptr;
  const bool ok = withRank(shapes.size(), [&](auto rank) {
    tensor = initTensorDescripter<decltype(rank)::value>(shapes, file, init, useFile, elementBytes);
  });
  if (!ok)
    std::fprintf(stderr, "Not support dim greater than 5.\n");
  return tensor;
}

void *GetFloatTensorDescripter(std::vector<size_t> &shapes, std::string file, bool init,
                               bool useFile) {
  return GetTensorDescripter(shapes, file, init, useFile, sizeof(float));
}

void SaveFloatTensor(ModelInfo *info, std::vector<void *> params, std::string &file) {
  auto &shapes = info->GetOutputSize(0);
  void *tensor = params[0];
  const size_t bytes = info->GetOutputNumElements(0) * info->ElementBytes();
  const bool ok = withRank(shapes.size(), [&](auto rank) {
    auto *t = reinterpret_cast<FloatTensor<decltype(rank)::value> *>(tensor);
    saveRaw(file, t->aligned, bytes);
  });
  if (!ok)
    std::fprintf(stderr, "Not support save dim greater than 5.\n");
}

std::vector<void *> GetParamsVec(ModelInfo *info) {
  std::vector<void *> params;
  for (size_t i = 0; i < info->OutputNums(); ++i)
    params.emplace_back(
        GetTensorDescripter(info->GetOutputSize(i), "", false, false, info->ElementBytes()));
  for (size_t i = 0; i < info->InputNums(); ++i)
    params.emplace_back(GetTensorDescripter(info->GetInputSize(i),
                                            info->ExistFile() ? info->GetFile(i) : "", true,
                                            info->ExistFile(), info->ElementBytes()));
  return params;
}

void *LoadLibrary(std::string libName) {
  void *handle = dlopen(libName.c_str(), RTLD_LAZY);
  if (!handle) {
    std::fprintf(stderr, "Failed to open library:%s\n", dlerror());
    return nullptr;
  }
  return handle;
}

RunGraphFuncPtr LoadFunc(void *handle, std::string funcName) {
  if (!handle)
    return nullptr;
  dlerror();
  RunGraphFuncPtr func = (RunGraphFuncPtr)dlsym(handle, funcName.c_str());
  const char *err = dlerror();
  if (err) {
    std::fprintf(stderr, "Failed to find run function: %s\n", err);
    return nullptr;
  }
  return func;
}

void RunGraphFunc(RunGraphFuncPtr func, std::vector<void *> &params) {
  if (!func)
    return;
  switch (params.size()) {
  case 0:
    func();
    break;
  case 1:
    func(params[0]);
    break;
  case 2:
    func(params[0], params[1]);
    break;
  case 3:
    func(params[0], params[1], params[2]);
    break;
  case 4:
    func(params[0], params[1], params[2], params[3]);
    break;
  case 5:
    func(params[0], params[1], params[2], params[3], params[4]);
    break;
  default:
    std::fprintf(stderr, "Not Support params more than 5.\n");
    break;
  }
}

void ClearOutputTensor(ModelInfo *info, std::vector<void *> &params) {
  for (size_t i = 0; i < info->OutputNums(); ++i) {
    const bool ok = withRank(info->GetOutputSize(i).size(), [&](auto rank) {
      reinterpret_cast<FloatTensor<decltype(rank)::value> *>(params[i])->clear();
    });
    if (!ok)
      std::fprintf(stderr, "Not support clear tensor which dim more than 5.\n");
  }
}

} // namespace multi_device
