// Adapter "tvm_arcfaceresnet100": serves the arcfaceresnet100 model (name kept from reference jobs/tvm_arcfaceresnet100/tvm_arcfaceresnet100.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMArcfaceresnet100Job, "arcfaceresnet100", "arcfaceresnet100-8")
