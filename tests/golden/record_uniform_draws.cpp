// Prints what the C++ standard library's generator gives for the draws the reference's
// init_matrix makes (reference test/test.hpp:36-38: std::mt19937 gen(1) and
// std::uniform_real_distribution<float> dis(-1.0f, 1.0f)), one value per line, exactly
// (hexadecimal float).  Uses nothing but <random>: it is the recipe behind
// "uniform_seed1_first6" in oracle_kat.json and lets any number of further draws be
// compared with the oracle's generator.
//
//   g++ -O1 -std=c++17 record_uniform_draws.cpp -o record_uniform_draws
//   ./record_uniform_draws <seed> <lo> <hi> <count>
#include <cstdio>
#include <cstdlib>
#include <random>

int main(int argc, char** argv)
{
    if(argc != 5)
    {
        std::fprintf(stderr, "usage: %s seed lo hi count\n", argv[0]);
        return 2;
    }
    std::mt19937                          gen(static_cast<unsigned>(std::strtoul(argv[1], nullptr, 10)));
    std::uniform_real_distribution<float> dis(std::strtof(argv[2], nullptr), std::strtof(argv[3], nullptr));
    const long                            count = std::strtol(argv[4], nullptr, 10);
    for(long i = 0; i < count; ++i)
    {
        std::printf("%a\n", static_cast<double>(dis(gen)));
    }
    return 0;
}
