// MFMA GEMM skeletons (filled in below)
#pragma once
