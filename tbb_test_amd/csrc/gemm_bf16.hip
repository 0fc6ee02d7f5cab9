// bf16 GEMM kernels (placeholder translation unit; the kernels are added with the bf16 model).
#include "kernels.h"
