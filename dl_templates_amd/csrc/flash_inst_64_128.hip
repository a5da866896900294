#define DLT_DK 64
#define DLT_DV 128
#include "flash_inst.hpp"
