// the reference's include path for what rg_mirror/collectors.h declares
#pragma once
#include "rg_mirror/collectors.h"
