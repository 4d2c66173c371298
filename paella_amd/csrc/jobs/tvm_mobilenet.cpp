// Adapter "tvm_mobilenet": serves the mobilenetv2 model (name kept from reference jobs/tvm_mobilenet/tvm_mobilenet.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMMobilenetJob, "mobilenetv2", "mobilenetv2-7")
