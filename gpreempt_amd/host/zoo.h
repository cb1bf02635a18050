// Native model builders (see zoo.cpp).
#pragma once
#include <string>
#include "model.h"

namespace foo {

// Fills `m` with the storages and kernels of `workload` ("name" or "name@key=value,...").
// Status::NotFound for an unknown name, Status::OutOfRange for a bad option.
Status zoo_build(Model &m, const std::string &workload);

}  // namespace foo
