// All gfx950 kernels of the per-column gradient quantizer (fp32, QWord = uint32); the overview of the work
// decomposition is at the top of quantizer_kernels_common.h.
#pragma once

#include "quantizer_kernels_common.h"
#include "quantizer_kernels_tile.h"
#include "quantizer_kernels_column.h"
#include "quantizer_kernels_register.h"
#include "quantizer_kernels_tall.h"
#include "quantizer_kernels_strip.h"
#include "quantizer_kernels_unquantize.h"
#include "quantizer_kernels_batch.h"
