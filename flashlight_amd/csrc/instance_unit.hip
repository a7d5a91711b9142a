// One kernel instance per translation unit so the instances build in parallel.
// The build passes -DFL_INST_NAME=<name> -DFL_INST_ARGS=<Dqk,Dv,RW,BN,NW,NS,FEAT> taken from instance_list.inc, once per
// element type.
#include "instances.h"

#ifndef FL_INST_NAME
#error "FL_INST_NAME / FL_INST_ARGS must be given on the command line"
#endif

// -DFL_INST_F16=1 compiles the instance for fp16 elements instead of bf16.
#if defined(FL_INST_F16) && FL_INST_F16
#define FL_EXPAND_DEF(NAME, ...) FL_INSTANCE_DEF(NAME, _f16, fl::f16_t, __VA_ARGS__)
#else
#define FL_EXPAND_DEF(NAME, ...) FL_INSTANCE_DEF(NAME, _bf16, fl::bf16_t, __VA_ARGS__)
#endif
FL_EXPAND_DEF(FL_INST_NAME, FL_INST_ARGS)
