// Adapter "tvm_squeezenet1_1": serves the squeezenet1_1 model (name kept from reference jobs/tvm_squeezenet1_1/tvm_squeezenet1_1.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMSqueezeNet11Job, "squeezenet1_1", "squeezenet1.1-7")
