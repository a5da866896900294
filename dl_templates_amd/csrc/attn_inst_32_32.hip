#define DLT_DK 32
#define DLT_DV 32
#include "attn_inst.hpp"
