#define DLT_D 64
#include "swa1_inst.hpp"
