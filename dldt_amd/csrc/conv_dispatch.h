// Epilogue flag word -> kernel instance: the hot step lists are template constants of the MFMA
// convolution kernels, everything else runs the instance that reads the flags at run time (kDyn).
#pragma once
#include "conv_epilogue.h"

// `core` (the flag word without CF_OUT_XOR) must be in scope; X(FLAGS, ...) is expanded with FLAGS a constant
#define HIPIE_FOR_EACH_EPILOGUE(X, ...)                                                      \
    switch (core) {                                                                          \
    case E_PLAIN0: X(E_PLAIN0, __VA_ARGS__); break;                                          \
    case E_PLAIN: X(E_PLAIN, __VA_ARGS__); break;                                            \
    case E_RESU8: X(E_RESU8, __VA_ARGS__); break;                                            \
    case E_RESF32: X(E_RESF32, __VA_ARGS__); break;                                          \
    case E_RESGEMM: X(E_RESGEMM, __VA_ARGS__); break;                                        \
    case E_F32: X(E_F32, __VA_ARGS__); break;                                                \
    case E_SCALE: X(E_SCALE, __VA_ARGS__); break;                                            \
    case E_SCALEFQ: X(E_SCALEFQ, __VA_ARGS__); break;                                        \
    case E_DEQFQ: X(E_DEQFQ, __VA_ARGS__); break;                                            \
    case E_GELUFQ: X(E_GELUFQ, __VA_ARGS__); break;                                          \
    case E_RESI8: X(E_RESI8, __VA_ARGS__); break;                                            \
    case E_F32RES: X(E_F32RES, __VA_ARGS__); break;                                          \
    case E_F32RELU: X(E_F32RELU, __VA_ARGS__); break;                                        \
    case E_CLAMPFQ: X(E_CLAMPFQ, __VA_ARGS__); break;                                        \
    case E_SCALEFQ0: X(E_SCALEFQ0, __VA_ARGS__); break;                                      \
    case E_PLAIN0 & ~CF_FQ_DIV2: X((E_PLAIN0 & ~CF_FQ_DIV2), __VA_ARGS__); break;            \
    case E_RESU8 & ~CF_FQ_DIV2: X((E_RESU8 & ~CF_FQ_DIV2), __VA_ARGS__); break;              \
    case E_RESGEMM & ~CF_FQ_DIV2: X((E_RESGEMM & ~CF_FQ_DIV2), __VA_ARGS__); break;          \
    case E_CLAMPFQ & ~CF_FQ_DIV2: X((E_CLAMPFQ & ~CF_FQ_DIV2), __VA_ARGS__); break;          \
    default: X(kDyn, __VA_ARGS__); break;                                                    \
    }

