// transpose4d_f / transpose2d_f (kernels.h:519-540): output axis a is input axis
// shuffle[a].  These are the layout ops an imported NCHW model needs at its
// boundary (NCHW2NHWC = {0,2,3,1}, NHWC2NCHW = {0,3,1,2}).
//
// A 32x33 LDS tile turns the permutation into coalesced reads AND coalesced
// writes whenever the input's innermost axis does not stay innermost: the tile
// spans (input innermost axis) x (the input axis that becomes the output's
// innermost).  When the innermost axis is unchanged a plain gather is already
// coalesced on both sides.
#include "common.hpp"

using namespace swc_hip;

namespace {

struct Perm4 {
    unsigned idim[4];      // input dims
    unsigned odim[4];      // output dims: odim[a] = idim[shuffle[a]]
    unsigned shuffle[4];
    size_t istride[4];     // element strides of the input axes
    size_t ostride_of_in[4];   // output stride of each INPUT axis
};

// innermost axis preserved: one thread per output element, linear in the output
__global__ __launch_bounds__(256) void permute_gather(const float *__restrict__ in, float *__restrict__ out, Perm4 p,
                                                      size_t total) {
    const size_t step = (size_t)gridDim.x * 256;
    for (size_t o = (size_t)blockIdx.x * 256 + threadIdx.x; o < total; o += step) {
        size_t r = o, src = 0;
#pragma unroll
        for (int a = 3; a >= 0; --a) {
            const unsigned i = (unsigned)(r % p.odim[a]);
            r /= p.odim[a];
            src += (size_t)i * p.istride[p.shuffle[a]];
        }
        out[o] = in[src];
    }
}

// Tiled: X = input axis 3 (contiguous in the input), Y = input axis `ya` that
// becomes the output's innermost axis.  blockIdx.x walks tiles of (X, Y),
// blockIdx.y the remaining two input axes.
__global__ __launch_bounds__(256) void permute_tiled(const float *__restrict__ in, float *__restrict__ out, Perm4 p,
                                                     int ya, int ra, int rb, unsigned tiles_x) {
    __shared__ float tile[32][33];
    const unsigned tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
    const unsigned x0 = (blockIdx.x % tiles_x) * 32, y0 = (blockIdx.x / tiles_x) * 32;
    const unsigned ia = blockIdx.y % p.idim[ra], ib = blockIdx.y / p.idim[ra];
    const size_t ibase = (size_t)ia * p.istride[ra] + (size_t)ib * p.istride[rb];
    const size_t obase = (size_t)ia * p.ostride_of_in[ra] + (size_t)ib * p.ostride_of_in[rb];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const unsigned y = y0 + ty + 8 * j, x = x0 + tx;
        if (y < p.idim[ya] && x < p.idim[3]) tile[ty + 8 * j][tx] = in[ibase + (size_t)y * p.istride[ya] + x];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const unsigned x = x0 + ty + 8 * j, y = y0 + tx;
        if (y < p.idim[ya] && x < p.idim[3])
            out[obase + (size_t)x * p.ostride_of_in[3] + (size_t)y * p.ostride_of_in[ya]] = tile[tx][ty + 8 * j];
    }
}

int permute(const char *who, const float *input, float *output, const size_t *idims, const size_t *odims,
            const size_t *shuffle, int nd) {
    if (!idims || !odims || !shuffle) return fail(SWC_HIP_EINVAL, "%s: null shape array", who);
    Perm4 p;
    // embed a 2-D problem as [1, 1, d0, d1]
    const int pad = 4 - nd;
    bool seen[4] = {false, false, false, false};
    size_t total = 1;
    for (int a = 0; a < 4; ++a) {
        const size_t id = a < pad ? 1 : idims[a - pad];
        const size_t sh = a < pad ? (size_t)a : shuffle[a - pad] + pad;
        if (id > 0xffffffffu || sh > 3 || seen[sh]) return fail(SWC_HIP_EINVAL, "%s: bad dims or shuffle", who);
        seen[sh] = true;
        p.idim[a] = (unsigned)id;
        p.shuffle[a] = (unsigned)sh;
        total *= id;
    }
    for (int a = 0; a < 4; ++a) {
        p.odim[a] = p.idim[p.shuffle[a]];
        const size_t od = a < pad ? 1 : odims[a - pad];
        if (od != p.odim[a]) return fail(SWC_HIP_EINVAL, "%s: odims[%d] is not idims[shuffle[%d]]", who, a - pad, a - pad);
    }
    if (total == 0) return SWC_HIP_OK;
    if (!input || !output) return fail(SWC_HIP_EINVAL, "%s: null pointer", who);
    if (input == output) return fail(SWC_HIP_EINVAL, "%s: in-place transpose is not supported", who);
    size_t s = 1;
    for (int a = 3; a >= 0; --a) {
        p.istride[a] = s;
        s *= p.idim[a];
    }
    s = 1;
    for (int a = 3; a >= 0; --a) {
        p.ostride_of_in[p.shuffle[a]] = s;
        s *= p.odim[a];
    }
    const int ya = (int)p.shuffle[3];   // input axis that becomes the output's innermost
    if (ya == 3) {
        size_t blocks = (total + 255) / 256;
        if (blocks > 65536) blocks = 65536;
        permute_gather<<<(unsigned)blocks, 256, 0, stream()>>>(input, output, p, total);
    } else {
        int rest[2], n = 0;
        for (int a = 0; a < 3; ++a)
            if (a != ya) rest[n++] = a;
        const unsigned tiles_x = (p.idim[3] + 31) / 32, tiles_y = (p.idim[ya] + 31) / 32;
        const size_t gy = (size_t)p.idim[rest[0]] * p.idim[rest[1]];
        if ((size_t)tiles_x * tiles_y > 0x7fffffffu || gy > 65535) {
            size_t blocks = (total + 255) / 256;
            if (blocks > 65536) blocks = 65536;
            permute_gather<<<(unsigned)blocks, 256, 0, stream()>>>(input, output, p, total);
        } else {
            permute_tiled<<<dim3(tiles_x * tiles_y, (unsigned)gy), 256, 0, stream()>>>(input, output, p, ya, rest[0],
                                                                                     rest[1], tiles_x);
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SWC_HIP_ERUNTIME, "%s: launch failed: %s", who, hipGetErrorString(e));
    return SWC_HIP_OK;
}

} // namespace

extern "C" {

int swc_hip_transpose4d_f(const float *input, float *output, const size_t *idims, const size_t *odims,
                          const size_t *shuffle) {
    SWC_REQUIRE_INIT();
    return permute("swc_hip_transpose4d_f", input, output, idims, odims, shuffle, 4);
}

int swc_hip_transpose2d_f(const float *input, float *output, const size_t *idims, const size_t *odims,
                          const size_t *shuffle) {
    SWC_REQUIRE_INIT();
    return permute("swc_hip_transpose2d_f", input, output, idims, odims, shuffle, 2);
}

} // extern "C"
