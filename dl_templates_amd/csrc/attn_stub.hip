#include "dlt_internal.hpp"
int dlt_attn_forward(const AttnProblem&, const AttnTensors&, hipStream_t) { return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention forward not built"); }
int dlt_attn_backward(const AttnProblem&, const AttnTensors&, hipStream_t) { return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention backward not built"); }
