// Declared in SpatiallySparseLayer.h; kept so that includes written for the
// reference resolve.
#pragma once
#include "SpatiallySparseLayer.h"
