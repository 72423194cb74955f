// The public API header lives in include/ (rocal_api_mi355x.h); this name is kept for the sources of the host layer.
#pragma once
#include "rocal_api_mi355x.h"
