#include "RowFusion.h"

namespace ThorImplementation {

void tryRowFusion(RowFusionContext&) {}

}  // namespace ThorImplementation
