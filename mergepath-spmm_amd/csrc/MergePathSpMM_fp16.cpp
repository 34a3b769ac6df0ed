// MergePathSpMM_fp16 <input_file> <dimension> <cost> <threads_per_wave> <repeat>
// fp16 values/features, fp32 accumulation (counterpart of src/MergePathSpMM_fp16.cu's main()).
#include "mergepath_driver.hpp"

int main(int argc, char **argv) { return drv::mergepath_main<uint16_t>(argc, argv); }
