#define DLT_DK 256
#define DLT_DV 256
#define DLT_ONE_PATCH
#include "attn_inst.hpp"
