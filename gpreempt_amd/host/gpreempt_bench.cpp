// Command-line front end of the scenario runner, in the shape of the reference's client
// programs (`blpclient config.json`, src/cuda-clients/blpclient.cpp:225-241):
//   gpreempt_bench config.json [policy]     -> JSON report on stdout
//   gpreempt_bench --probe <workload> [trials]
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>
#include "harness.h"

int main(int argc, char **argv) {
    if (argc < 2) {
        std::cout << "Usage: " << argv[0] << " config.json [policy] | --probe workload [trials] [0 = all kernels at once | 1 = as one program | 2 = kernel by kernel, bounded queue (default)]" << std::endl;
        return -1;
    }
    std::string report;
    if (std::strcmp(argv[1], "--probe") == 0 && argc >= 3) {
        Status s = foo::preempt_probe(argv[2], argc > 3 ? std::atoi(argv[3]) : 200, argc > 4 ? std::atoi(argv[4]) : 2, 1, report);
        std::cout << report << std::endl;
        return s == Status::Succ ? 0 : 1;
    }
    std::ifstream f(argv[1]);
    if (!f.is_open()) { std::cerr << "cannot open " << argv[1] << std::endl; return 1; }
    std::stringstream ss;
    ss << f.rdbuf();
    std::string cfg = ss.str();
    if (argc > 2) {  // policy override: a later duplicate key wins, so append it before the closing brace
        size_t b = cfg.rfind('}');
        if (b != std::string::npos) cfg.insert(b, std::string(",\"policy\":\"") + argv[2] + "\"");
    }
    Status s = foo::run_scenario(cfg, report);
    std::cout << report << std::endl;
    return s == Status::Succ ? 0 : 1;
}
