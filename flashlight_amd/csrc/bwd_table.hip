// Table of the compiled backward kernels (host data only).
#include "bwd_instances.h"

FL_BWD_LIST(FL_BWD_DECL)

namespace fl {
const BwdInstance kBwdInstances[] = {FL_BWD_LIST(FL_BWD_ROW)};
const int kNumBwdInstances = sizeof(kBwdInstances) / sizeof(kBwdInstances[0]);
}  // namespace fl
