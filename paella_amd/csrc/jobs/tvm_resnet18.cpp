// Adapter "tvm_resnet18": serves the resnet18 model (name kept from reference jobs/tvm_resnet18/tvm_resnet18.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMResnet18Job, "resnet18", "resnet18-v2-7")
