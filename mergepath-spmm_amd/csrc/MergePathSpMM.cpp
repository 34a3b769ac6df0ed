// MergePathSpMM <input_file> <dimension> <cost> <threads_per_wave> <repeat>
// fp32 merge-path SpMM driver (counterpart of src/MergePathSpMM.cu's main()).
#include "mergepath_driver.hpp"

int main(int argc, char **argv) { return drv::mergepath_main<float>(argc, argv); }
