#include "kernel_manager.h"
namespace es
{
std::shared_ptr<plan_t> plan_contraction(einsummable_t const&, int) { return nullptr; }
}  // namespace es
