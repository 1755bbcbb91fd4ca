// The slice of the reference's executor settings that the hot path consumes:
// the backend selector (runtime/executor/executor_settings_base.h:31-49, with a
// new value for this executor, which is where EngineImpl's backend switch,
// runtime/core/engine_impl.cc:93-96,122-125, would pick it up), the activation
// data type (:54-66) and LlmExecutorSettings' KV capacity
// (runtime/executor/llm_executor_settings.h:95-154, max_num_tokens :140-142).
#ifndef LITERT_LM_AMD_EXECUTOR_LLM_EXECUTOR_SETTINGS_H_
#define LITERT_LM_AMD_EXECUTOR_LLM_EXECUTOR_SETTINGS_H_

#include <string>

#include "status.h"

namespace litert::lm {

enum class Backend { CPU_ARTISAN, GPU_ARTISAN, CPU, GPU, GOOGLE_TENSOR_ARTISAN, QNN, GPU_HIP };

inline StatusOr<Backend> GetBackendFromString(const std::string& s) {
  if (s == "cpu_artisan") return Backend::CPU_ARTISAN;
  if (s == "gpu_artisan") return Backend::GPU_ARTISAN;
  if (s == "cpu") return Backend::CPU;
  if (s == "gpu") return Backend::GPU;
  if (s == "google_tensor_artisan") return Backend::GOOGLE_TENSOR_ARTISAN;
  if (s == "qnn") return Backend::QNN;
  if (s == "hip") return Backend::GPU_HIP;
  return InvalidArgumentError("Unsupported backend: " + s +
                              ". Supported backends are: [cpu_artisan, gpu_artisan, cpu, gpu, "
                              "google_tensor_artisan, qnn, hip]");
}

enum class ActivationDataType { FLOAT32, FLOAT16, INT16, INT8 };

class LlmExecutorSettings {
 public:
  static StatusOr<LlmExecutorSettings> CreateDefault(Backend backend) {
    if (backend != Backend::GPU_HIP)
      return InvalidArgumentError("This build only provides the hip backend of the executor.");
    LlmExecutorSettings s;
    s.backend_ = backend;
    return s;
  }
  Backend GetBackend() const { return backend_; }
  // Capacity of the KV cache in tokens; 0 means "not set" as in the reference.
  int GetMaxNumTokens() const { return max_num_tokens_; }
  void SetMaxNumTokens(int n) { max_num_tokens_ = n; }
  int GetMaxNumImages() const { return max_num_images_; }
  void SetMaxNumImages(int n) { max_num_images_ = n; }
  ActivationDataType GetActivationDataType() const { return activation_; }
  void SetActivationDataType(ActivationDataType t) { activation_ = t; }
  const std::string& GetCacheDir() const { return cache_dir_; }
  void SetCacheDir(std::string d) { cache_dir_ = std::move(d); }
  int GetDevice() const { return device_; }
  void SetDevice(int d) { device_ = d; }

 private:
  Backend backend_ = Backend::GPU_HIP;
  int max_num_tokens_ = 0;
  int max_num_images_ = 0;
  ActivationDataType activation_ = ActivationDataType::FLOAT32;
  std::string cache_dir_;
  int device_ = 0;
};

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_LLM_EXECUTOR_SETTINGS_H_
