#include "utils.h"
#include "TurboFNO.h"
#include <fstream>
#include <sstream>

int ntest = 5;
int threadblock_bs = 4;

std::vector<int> parse_line(const std::string& line)
{
    std::istringstream in(line);
    std::string key, eq;
    in >> key >> eq;
    std::vector<int> out;
    for (int v; in >> v;) out.push_back(v);
    return out;
}

std::map<std::string, std::vector<int>> load_problem_config(const std::string& path)
{
    std::map<std::string, std::vector<int>> cfg;
    std::ifstream f(path);
    for (std::string line; std::getline(f, line);) {
        if (line.empty() || line[0] == '#') continue;
        std::istringstream in(line);
        std::string key;
        in >> key;
        cfg[key] = parse_line(line);
    }
    return cfg;
}

void generate_random_vector(float* target, long n)
{
    for (long i = 0; i < n; ++i) {
        float v = (float)(rand() % 10) * 0.001f;
        target[i] = (rand() % 2 == 0) ? v : -v;
    }
}
