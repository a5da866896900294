#define DLT_SWA2_D 64
#include "swa2_inst.hpp"
