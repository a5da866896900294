#define DLT_DK 64
#define DLT_DV 128
#include "attn_inst.hpp"
