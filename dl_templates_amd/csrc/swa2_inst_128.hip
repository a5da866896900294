#define DLT_SWA2_D 128
#include "swa2_inst.hpp"
