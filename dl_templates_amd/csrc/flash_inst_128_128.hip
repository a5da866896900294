#define DLT_DK 128
#define DLT_DV 128
#include "flash_inst.hpp"
