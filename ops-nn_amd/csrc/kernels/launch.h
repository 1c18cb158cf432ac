// Internal: kernel-variant ids shared by the launchers and the selector.
#pragma once
#include "opsnn_kernels.h"

#define OPSNN_NOT_TAKEN 0x7fff0001

enum {
    OPSNN_VARIANT_AUTO = 0,
    OPSNN_VARIANT_PLAIN = 1,      // strided one-thread-per-output kernels (any shape)
    OPSNN_VARIANT_I8_256 = 2,     // int8 MFMA, 256x256 tile
    OPSNN_VARIANT_I8_128 = 3,     // int8 MFMA, 128x128 tile
};
