// The class this header declared in the reference now lives in operator.h.
#pragma once
#include "mirage/threadblock/operator.h"
