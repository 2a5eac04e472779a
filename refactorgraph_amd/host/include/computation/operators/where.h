// the reference's include path for what rg_mirror/computation.h declares
#pragma once
#include "rg_mirror/computation.h"
