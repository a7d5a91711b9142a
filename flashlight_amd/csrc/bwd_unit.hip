// Backward kernels of one (head dim, feature set); the build passes -DFL_BWD_D=<D> -DFL_BWD_FEAT=<bits>.
#include "bwd_instances.h"

#if !defined(FL_BWD_D) || !defined(FL_BWD_FEAT)
#error "FL_BWD_D / FL_BWD_FEAT must be given on the command line"
#endif

#define FL_BWD_EXPAND(D, FEAT) FL_BWD_DEF(D, FEAT)
FL_BWD_EXPAND(FL_BWD_D, FL_BWD_FEAT)
