// CPU check of the drivers' config-file grammar (turbofno_amd/host/utils.cpp): prints the parsed
// lists as "key:v,v,v;" in key order so the Python test can compare them.
#include "../../turbofno_amd/host/utils.h"
#include <iostream>
int main(int argc, char** argv)
{
    auto cfg = load_problem_config(argc > 1 ? argv[1] : "");
    for (auto& kv : cfg) {
        std::cout << kv.first << ":";
        for (size_t i = 0; i < kv.second.size(); ++i) std::cout << (i ? "," : "") << kv.second[i];
        std::cout << ";";
    }
    std::cout << "\n";
    return 0;
}
