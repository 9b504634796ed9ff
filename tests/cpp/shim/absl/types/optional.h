// Front-end stand-in for <absl/types/optional.h>: see ../../README.md.
#pragma once
#include <optional>
namespace absl {
using std::optional;
using std::nullopt;
using std::nullopt_t;
using std::make_optional;
}  // namespace absl
