// Internal glue: the public C ABI constants plus launch helpers.
#pragma once
#include "../../include/lcq.h"
