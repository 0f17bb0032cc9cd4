/* csr2csc.h -- the reference's include/csr2csc.h:9-13 (csr2csc, csc2csr), served by
 * MatXtract.h; a driver that includes "csr2csc.h" as the reference's does finds them here. */
#ifndef MATXTRACT_CSR2CSC_H
#define MATXTRACT_CSR2CSC_H
#include "MatXtract.h"
#endif
