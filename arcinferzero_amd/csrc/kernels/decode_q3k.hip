// "decode" module, part: the LDS-staged GEMV kernels (gemv, gemv_mt) for GGUF type 11 (Q3_K).
#include "common.h"
template <int QT> struct UnitsPerSb { static constexpr int v = QT == QT_Q8_0 ? 16 : 8; };
#define GEMV_LDS_QT 11
#include "gemv_lds.inc"
