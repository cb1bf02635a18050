// Multi-tenant scenario runner and the per-kernel preemption probe (see harness.cpp).
#pragma once
#include <cstdint>
#include <string>
#include "util/common.h"

namespace foo {

// Runs the task file `config_text` (DISB schema plus "policy": "wb" | "wb-async" | "wb-chunk" | "wb-chunk-async" | "np" | "seq" |
// "lco", "standalone_runs", "warmups", "hp_requests", "pre_preempt_hint_us") and writes a JSON report.
Status run_scenario(const std::string &config_text, std::string &report_text);

// Measures flag-store -> stream-drained latency of `workload` per stopped kernel.
Status preempt_probe(const std::string &workload, int trials, int use_graph, uint64_t seed, std::string &report_text);

}  // namespace foo
