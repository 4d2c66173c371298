// Adapter "tvm_resnet34": serves the resnet34 model (name kept from reference jobs/tvm_resnet34/tvm_resnet34.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMResnet34Job, "resnet34", "resnet34-v2-7")
