// Elementwise kernels of the layer that routes rows to the quantized linears (include/fe_route.h): SwiGLU on the bf16
// outputs of gate and up, and the strided row copy that places decode rows into a fused projection's layout.
#include "kcommon.h"

// out[r][c] = bf16(bf16(silu(gate[r][c])) * up[r][c]); gate / up rows share stride ld, out is [rows][inter]; a thread
// takes 2 columns. grid (ceil(inter / 2 / 256), rows), 256 threads. (kernels/k-core/src/misc.rs:58-71)
extern "C" __global__ __launch_bounds__(256) void fe_silu_mul(uint16_t* out, const uint16_t* gate, const uint16_t* up,
                                                              uint32_t ld, uint32_t inter) {
    const uint32_t r = blockIdx.y, c = (blockIdx.x * 256 + threadIdx.x) * 2;
    if (c >= inter) return;
    const uint32_t g = *(const uint32_t*)(gate + (size_t)r * ld + c), u = *(const uint32_t*)(up + (size_t)r * ld + c);
    *(uint32_t*)(out + (size_t)r * inter + c) = silu_mul_bf16x2(g, u);
}

// dst[r][c .. c + 1] = src[r][c .. c + 1]. grid (rows, ceil(cols / 2 / 256)), 256 threads.
// (kernels/k-core/src/misc.rs:164-171)
extern "C" __global__ __launch_bounds__(256) void fe_copy2d(uint16_t* dst, uint32_t ldd, const uint16_t* src, uint32_t lds,
                                                            uint32_t cols) {
    const uint32_t r = blockIdx.x, c = (blockIdx.y * 256 + threadIdx.x) * 2;
    if (c < cols) *(uint32_t*)(dst + (size_t)r * ldd + c) = *(const uint32_t*)(src + (size_t)r * lds + c);
}
