#define DLT_D 128
#include "swa1_inst.hpp"
