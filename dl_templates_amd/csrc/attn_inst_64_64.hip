#define DLT_DK 64
#define DLT_DV 64
#include "attn_inst.hpp"
