// Adapter "tvm_mnist": serves the mnist model (name kept from reference jobs/tvm_mnist/tvm_mnist.cpp so existing
// client command lines keep working; there is no TVM underneath).
#include "models/model_job.h"

PAELLA_DEFINE_MODEL_JOB(TVMMnistJob, "mnist", "mnist-8")
