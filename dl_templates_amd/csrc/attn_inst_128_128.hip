#define DLT_DK 128
#define DLT_DV 128
#include "attn_inst.hpp"
