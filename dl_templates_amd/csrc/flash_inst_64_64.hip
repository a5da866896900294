#define DLT_DK 64
#define DLT_DV 64
#include "flash_inst.hpp"
