// Adapter "tvm_ultraface320": serves the ultraface320 model (name kept from reference jobs/tvm_ultraface320/tvm_ultraface320.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMUltraface320Job, "ultraface320", "ultraface320")
