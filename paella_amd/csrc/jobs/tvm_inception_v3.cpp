// Adapter "tvm_inception_v3": serves the inception_v3 model (name kept from reference jobs/tvm_inception_v3/tvm_inception_v3.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMInceptionV3Job, "inception_v3", "inception_v3")
