// Adapter "tvm_resnet50": serves the resnet50 model (name kept from reference jobs/tvm_resnet50/tvm_resnet50.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMResnet50, "resnet50", "resnet50-v2-7")
