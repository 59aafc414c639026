// Part of the public API, declared in SparseConvNetAPI.h; this header keeps
// the include name drivers written for the reference use.
#pragma once
#include "SparseConvNetAPI.h"
