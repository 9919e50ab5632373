// Shape of the prefill attention workgroup, shared by the kernels and the entry point that tells the host
// how many query rows one tile holds.
#pragma once
#ifndef PF_WAVES
#define PF_WAVES 8  // waves per workgroup
#endif
#ifndef PF_QT
#define PF_QT 1     // tiles of 16 query rows per wave
#endif
#define PF_ROWS (PF_WAVES * PF_QT * 16)
#define PF_THREADS (PF_WAVES * 64)
