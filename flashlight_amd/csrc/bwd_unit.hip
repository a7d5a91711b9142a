// Backward kernels of one (head dim, feature set); the build passes -DFL_BWD_D=<D> -DFL_BWD_FEAT=<bits>.
#include "bwd_instances.h"

#if !defined(FL_BWD_D) || !defined(FL_BWD_FEAT)
#error "FL_BWD_D / FL_BWD_FEAT must be given on the command line"
#endif

// -DFL_INST_F16=1 compiles the kernels for fp16 elements instead of bf16.
#if defined(FL_INST_F16) && FL_INST_F16
#define FL_BWD_EXPAND(D, FEAT) FL_BWD_DEF(D, FEAT, _f16, fl::f16_t)
#else
#define FL_BWD_EXPAND(D, FEAT) FL_BWD_DEF(D, FEAT, _bf16, fl::bf16_t)
#endif
FL_BWD_EXPAND(FL_BWD_D, FL_BWD_FEAT)
