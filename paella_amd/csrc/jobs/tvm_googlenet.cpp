// Adapter "tvm_googlenet": serves the googlenet model (name kept from reference jobs/tvm_googlenet/tvm_googlenet.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMGooglenetJob, "googlenet", "googlenet-9")
