#include "tc/autotuner/autotuner.h"

namespace tc {
namespace autotune {
namespace detail {
std::atomic<int> tunerSignal{0};
} // namespace detail
} // namespace autotune
} // namespace tc
