build_tl0/hip/ring_probe.hsaco: hip/ring_probe.hip hip/direct_dispatch.h \
  ../../include/paella_hip.h ../../include/paella_ops.h \
  ../../include/paella_ring.h \
  ../../include/llis/ipc/shm_primitive_channel.h \
  ../../include/llis/utils/gpu.h \
  ../../include/llis/job/finished_block_notifier.h \
  ../../include/llis/job/instrument_info.h ../../include/llis/ipc/defs.h \
  ../../include/llis/job/instrument.h
hip/direct_dispatch.h:
../../include/paella_hip.h:
../../include/paella_ops.h:
../../include/paella_ring.h:
../../include/llis/ipc/shm_primitive_channel.h:
../../include/llis/utils/gpu.h:
../../include/llis/job/finished_block_notifier.h:
../../include/llis/job/instrument_info.h:
../../include/llis/ipc/defs.h:
../../include/llis/job/instrument.h:
