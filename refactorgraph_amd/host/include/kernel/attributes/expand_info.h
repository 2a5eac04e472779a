// the reference's include path for what rg_mirror/attributes.h declares
#pragma once
#include "rg_mirror/attributes.h"
