#define DLT_DK 32
#define DLT_DV 32
#include "flash_inst.hpp"
