// Table of every compiled kernel instance (rows come from instance_list.inc).
#include "instances.h"

#define X(...) FL_INSTANCE_DECL(__VA_ARGS__)
#include "instance_list.inc"
#undef X

namespace fl {
const Instance kInstances[] = {
#define X(...) FL_INSTANCE_ROW(__VA_ARGS__)
#include "instance_list.inc"
#undef X
};
const int kNumInstances = sizeof(kInstances) / sizeof(kInstances[0]);
}  // namespace fl
