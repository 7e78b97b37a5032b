// Allocation-free split-K GEMM: cubert_op_gemm_splitk_noalloc.
//
// Y[M, N] (float32) = X[M, K] * W[N, K]^T + bias[N], with K shared by `splits` workgroups per
// tile.  The same kernels as cubert_op_gemm with CUBERT_SPLITS(n), whose caller has to bring a
// result buffer of n * M * N floats and add the parts up itself; here the partial sums live in
// a device array that is part of the library image, and a second kernel adds them into Y.  The
// call issues no hipMalloc / hipFree and no allocating library routine, so it can be used by
// code that must not allocate: under hipGraph capture, in a serving loop, in a harness that
// forbids allocation.
//
// The array (kScratchBytes, fixed) exists once per GPU the library image is loaded on and is held
// until the process ends.  Every call on a GPU uses that GPU's array: calls that overlap in time
// on one GPU (different streams, different threads) race on it.  Each call overwrites every
// partial sum it later reads, so nothing has to be cleared between calls.
#include <mutex>

#include "../../include/cubert.h"
#include "kernels.h"

namespace {

constexpr size_t kScratchBytes = 16u << 20;      // e.g. 2 parts of a 1600 x 1024 result, or 8 of 200 x 1024 (x 2)
constexpr int kMaxDevices = 64;

// The partial sums.  In host code this name is only a handle for hipGetSymbolAddress; the
// device address of each GPU's copy is looked up once per GPU and kept in g_scratch.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

std::mutex g_mutex;
float* g_scratch[kMaxDevices] = {};

// Address of the current device's copy of `scratch` (looked up on the first call per device).
bool scratch_of_current_device(float** out) {
    int dev = -1;
    CUBERT_HIP_OK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) {
        cubert::set_error("allocation-free GEMM: device ordinal " + std::to_string(dev) + " is not supported");
        return false;
    }
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_scratch[dev]) {
        void* p = nullptr;
        CUBERT_HIP_OK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) { cubert::set_error("allocation-free GEMM: the scratch array has no device address"); return false; }
        g_scratch[dev] = static_cast<float*>(p);
    }
    *out = g_scratch[dev];
    return true;
}

typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// y[i] = ((part 0 + part 1) + part 2) + ...   over n4 float quads; parts are `stride4` quads apart.
__global__ __launch_bounds__(256) void sum_parts_kernel(const f32x4_t* __restrict__ parts, f32x4_t* __restrict__ y,
                                                        size_t n4, size_t stride4, int nparts) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
        f32x4_t s = parts[i];
        for (int p = 1; p < nparts; ++p) s += parts[i + (size_t)p * stride4];
        y[i] = s;
    }
}

}  // namespace

namespace cubert {

// Called by Model::init so that a process that creates a model has the address before it
// starts capturing graphs; the entry point below looks it up itself otherwise.
bool noalloc_setup_current_device() {
    float* p = nullptr;
    return scratch_of_current_device(&p);
}

}  // namespace cubert

extern "C" {

size_t cubert_noalloc_scratch_bytes(void) { return kScratchBytes; }

int cubert_op_gemm_splitk_noalloc(const void* X, const void* W, const float* bias, float* Y, int M, int N, int K,
                                  int ldx, int elt, int splits, int tile, int flags, void* stream) {
    cubert::set_error("");
    if (splits < 1 || splits > 16) { cubert::set_error("allocation-free GEMM: splits must be 1..16"); return 1; }
    if (M <= 0 || N <= 0 || K <= 0) { cubert::set_error("allocation-free GEMM: empty problem"); return 1; }
    if (!Y || (reinterpret_cast<uintptr_t>(Y) & 15)) { cubert::set_error("allocation-free GEMM: Y must be 16-byte aligned"); return 1; }
    if (flags & ~(CUBERT_X_PACKED | CUBERT_W_PACKED)) {
        cubert::set_error("allocation-free GEMM: only the operand layout flags are accepted");
        return 1;
    }
    const size_t need = (size_t)splits * M * N * sizeof(float);
    if (splits > 1 && need > kScratchBytes) {
        cubert::set_error("allocation-free GEMM: splits * M * N floats = " + std::to_string(need) +
                          " bytes exceed the built-in scratch of " + std::to_string(kScratchBytes) + " bytes");
        return 1;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    cubert::GemmParams p;
    p.X = X; p.W = W; p.bias = bias; p.M = M; p.N = N; p.K = K; p.ldx = ldx; p.elt = elt;
    p.out_elt = cubert::kF32; p.epilogue = cubert::kEpiBias; p.tile = tile; p.splits = splits;
    p.x_packed = (flags & CUBERT_X_PACKED) != 0;
    p.w_packed = (flags & CUBERT_W_PACKED) != 0;
    if (splits == 1) {
        p.Y = Y;
        return cubert::launch_gemm(p, st) ? 0 : 1;
    }
    float* parts = nullptr;
    if (!scratch_of_current_device(&parts)) return 1;
    p.Y = parts;                                      // part z at parts + z * M * N
    if (!cubert::launch_gemm(p, st)) return 1;
    const size_t n4 = (size_t)M * N / 4;              // launch_gemm has checked N % 4 == 0
    const size_t blocks = (n4 + 255) / 256;
    hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)(blocks < 2048 ? blocks : 2048)), dim3(256), 0, st,
                       reinterpret_cast<const f32x4_t*>(parts), reinterpret_cast<f32x4_t*>(Y), n4, n4, splits);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { cubert::set_error(std::string("sum_parts_kernel launch failed: ") + hipGetErrorString(e)); return 1; }
    return 0;
}

}  // extern "C"
