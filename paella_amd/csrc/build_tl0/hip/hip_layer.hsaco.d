build_tl0/hip/hip_layer.hsaco: hip/hip_layer.hip \
  ../../include/paella_hip.h
../../include/paella_hip.h:
