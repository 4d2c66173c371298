// Adapter "tvm_densenet121": serves the densenet121 model (name kept from reference jobs/tvm_densenet121/tvm_densenet121.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMDensenet121Job, "densenet121", "densenet-9")
