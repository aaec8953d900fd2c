// tiling.h -- kept so that sources written against the reference's header set compile
// unchanged; everything on the GEMM path is declared in cake.h.
#pragma once
#include "cake.h"
