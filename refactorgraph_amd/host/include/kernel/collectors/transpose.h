// reference include path -> host mirror
#pragma once
#include "rg_mirror/collectors.h"
