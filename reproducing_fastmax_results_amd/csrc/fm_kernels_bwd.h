#pragma once
#include "fm_kernels.h"
