#pragma once
// int8 MFMA GEMM skeleton (filled in below).
