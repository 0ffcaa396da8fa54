// cascade_sa <text-file> <suffix-array-file> [key-words]
// The reference's command-line builder (src/main.cu:12-46) over the MI355X partition sort: the text (16-bit symbols) is
// one partition, the suffix array leaves as 5-byte little-endian entries. Host code only; everything on the device
// happens behind the C ABI.
#include "../../include/cascade_gpu_saca.hpp"

#include <chrono>

// every member of the builder class is compiled with the program, the per-partition members that it does not call included
template class cascade_hip::GPU_SACA<std::uint16_t>;

int main(int argc, char** argv)
{
    using T_sym_ = std::uint16_t;
    if (argc < 3) {
        std::cerr << "Usage: " << argv[0] << " <text-file> <suffix-array-file> [key-words]. Aborting.\n";
        std::exit(EXIT_FAILURE);
    }
    const std::string ip_path(argv[1]);
    const std::string op_path(argv[2]);
    const int key_words = argc > 3 ? std::atoi(argv[3]) : 1;

    cascade_hip::GPU_SACA<T_sym_> saca(ip_path, op_path, key_words);
    const auto t_0 = std::chrono::steady_clock::now();
    saca.build_SA();
    const auto t_1 = std::chrono::steady_clock::now();
    std::cerr << "Time taken: " << std::chrono::duration<double>(t_1 - t_0).count() << "s.\n";
    const csa_stats& st = saca.stats();
    std::cerr << "Suffixes: " << st.n << ", generations: " << st.generations << ", device time: " << st.ms_total << " ms.\n";
    return 0;
}
