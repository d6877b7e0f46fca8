// TEST INFRASTRUCTURE.  Stand-in for include/api/kernel_api.h, cut down to what a provider kernel touches: the three
// life-cycle calls the runtime makes and the protected tensor lists (reference: MSKernel :29-140, IKernel :143-166).
#ifndef TESTS_LITE_STUB_INCLUDE_API_KERNEL_API_H_
#define TESTS_LITE_STUB_INCLUDE_API_KERNEL_API_H_
#include <map>
#include <string>
#include <vector>

#include "include/api/status.h"
#include "include/api/types.h"

namespace mindspore {
class Context;
namespace kernel {
class MSKernel {
 public:
  virtual ~MSKernel() = default;
  virtual int Prepare() = 0;
  virtual int ReSize() = 0;
  virtual int Execute() = 0;
  // the session's config file sections (Model::LoadConfig / UpdateConfig), handed over by the scheduler after the
  // creator has run (scheduler.cc:1455-1457)
  void SetConfig(const std::map<std::string, std::map<std::string, std::string>> *config) { config_ = config; }
  std::map<std::string, std::string> GetConfig(const std::string &section) const {
    if (config_ == nullptr) return {};
    const auto it = config_->find(section);
    return it == config_->end() ? std::map<std::string, std::string>() : it->second;
  }

 protected:
  MSKernel() = default;
  MSKernel(const std::vector<MSTensor> &in, const std::vector<MSTensor> &out, const Context *ctx)
      : context_(ctx), inputs_(in), outputs_(out) {}
  const Context *context_ = nullptr;
  std::vector<MSTensor> inputs_, outputs_;
  const std::map<std::string, std::map<std::string, std::string>> *config_ = nullptr;
};

template <typename Primitive>
class IKernel : public MSKernel {
 protected:
  IKernel() = default;
  IKernel(const std::vector<MSTensor> &in, const std::vector<MSTensor> &out, const Primitive *primitive,
          const Context *ctx)
      : MSKernel(in, out, ctx), primitive_(primitive) {}
  const Primitive *primitive_ = nullptr;
};
}  // namespace kernel
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_KERNEL_API_H_
