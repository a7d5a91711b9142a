// One kernel instance per translation unit so the instances build in parallel.
// The build passes -DFL_INST_NAME=<name> -DFL_INST_ARGS=<Dqk,Dv,RW,BN,NW,FEAT> taken from instance_list.inc.
#include "instances.h"

#ifndef FL_INST_NAME
#error "FL_INST_NAME / FL_INST_ARGS must be given on the command line"
#endif

#define FL_EXPAND_DEF(NAME, ...) FL_INSTANCE_DEF(NAME, __VA_ARGS__)
FL_EXPAND_DEF(FL_INST_NAME, FL_INST_ARGS)
