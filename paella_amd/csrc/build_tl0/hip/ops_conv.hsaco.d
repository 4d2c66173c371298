build_tl0/hip/ops_conv.hsaco: hip/ops_conv.hip ../../include/paella_ops.h \
  ../../include/llis/job/finished_block_notifier.h \
  ../../include/llis/ipc/shm_primitive_channel.h \
  ../../include/llis/utils/gpu.h \
  ../../include/llis/job/instrument_info.h ../../include/llis/ipc/defs.h \
  hip/launch.h hip/direct_dispatch.h hip/pack.h hip/out_store.h \
  hip/pool_body.h hip/dense_body.h
../../include/paella_ops.h:
../../include/llis/job/finished_block_notifier.h:
../../include/llis/ipc/shm_primitive_channel.h:
../../include/llis/utils/gpu.h:
../../include/llis/job/instrument_info.h:
../../include/llis/ipc/defs.h:
hip/launch.h:
hip/direct_dispatch.h:
hip/pack.h:
hip/out_store.h:
hip/pool_body.h:
hip/dense_body.h:
