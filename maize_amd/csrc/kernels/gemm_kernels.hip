// Single translation unit of the gfx950 code object embedded in libmaize_hip.so.
#include "common.hpp"
#include "gemm_wave32.hpp"
#include "gemm_mt256.hpp"
#include "gemm_mt256_f8.hpp"
#include "gemm_skinny.hpp"
#include "splitk_reduce.hpp"
#include "pack.hpp"
#include "probes.hpp"
