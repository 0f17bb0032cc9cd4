/* mmio.h -- the reference's include/mmio.h:165-179 (mmio_allinone, exclusive_scan), served by
 * MatXtract.h; a driver that includes "mmio.h" as the reference's does finds them here. */
#ifndef MATXTRACT_MMIO_H
#define MATXTRACT_MMIO_H
#include "MatXtract.h"
#endif
