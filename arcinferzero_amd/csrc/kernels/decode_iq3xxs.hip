// "decode" module, part: the LDS-staged GEMV kernels (gemv, gemv_mt) for GGUF type 18 (IQ3_XXS).
#include "common.h"
template <int QT> struct UnitsPerSb { static constexpr int v = QT == QT_Q8_0 ? 16 : 8; };
#define GEMV_LDS_QT 18
#include "gemv_lds.inc"
