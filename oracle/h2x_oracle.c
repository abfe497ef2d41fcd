/*
 * h2x_oracle.c -- CPU restatement of the reference algorithms of DistConv's
 * non-convolution hot path (batch-norm statistics forward/backward, channel
 * softmax, halo pack/unpack, tensor-shuffler pack/unpack).
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the GPU library is compared
 * against and the CPU baseline a benchmark reports next to the GPU numbers.
 * Nothing in the product (the HIP library, its host-side layer classes, its
 * Python binding) may call, link or import it.
 *
 * Each function names the reference file:line it follows (paths relative to
 * the reference checkout).  What pins each function besides reading the
 * reference is listed in oracle/README.md.  PARITY UNPINNED: the FLT_MIN
 * clamp, the y > FLT_MIN guard and the FLT_MIN initial maximum of channel
 * softmax, and the sqrt(FLT_MIN) clamp and guard of instance softmax -- the
 * reference holds no softmax test or vector; everything else of softmax is
 * pinned by the textbook routine.
 *
 * Build: see oracle/Makefile (gcc -O3 -fopenmp, -ffp-contract=off so that the
 * only fused multiply-adds are the ones written explicitly).
 */
#include <float.h>
#include <math.h>
#include <omp.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define T float
#define SFX f32
#define T_MIN FLT_MIN
#define T_EXP expf
#define T_SQRT sqrtf
#define T_FMA fmaf
#include "h2x_oracle_impl.inc"
#undef T
#undef SFX
#undef T_MIN
#undef T_EXP
#undef T_SQRT
#undef T_FMA

#define T double
#define SFX f64
#define T_MIN DBL_MIN
#define T_EXP exp
#define T_SQRT sqrt
#define T_FMA fma
#include "h2x_oracle_impl.inc"
#undef T
#undef SFX
#undef T_MIN
#undef T_EXP
#undef T_SQRT
#undef T_FMA

#define ORC_MAX_DIMS 6

/* OpenMP threads the parallel loops of this file use. */
int orc_num_threads(void)
{
    return omp_get_max_threads();
}

/*
 * Destination rank and offset inside that rank's chunk of the packed buffer
 * for one local index.  Follows TensorMPIShuffler::find_destination,
 * legacy/include/distconv/tensor/shuffle_mpi.hpp:628-686 (device twin:
 * legacy/src/tensor/shuffle_mpi_cuda.cu:42-98), including the "-1" encoding
 * of evenly partitioned dimensions (DISTCONV_OPTIMIZE_FIND_DESTINATION).
 */
static void find_destination(int nd, const int64_t* local_idx, const int64_t* local_shape,
                             const int64_t* peer_locale_shape, const int32_t* rank_limits,
                             int* dst_rank, size_t* dst_offset)
{
    int rank = 0, rank_dim_offset = 1, rl = 0;
    size_t off = 0, lin = 1;
    for (int i = 0; i < nd; ++i)
    {
        int rank_idx, buffer_offset, buffer_dim;
        if (rank_limits[rl] == -1)
        {
            const int64_t g = local_idx[i] + rank_limits[rl + 1];
            const int d = rank_limits[rl + 2];
            rank_idx = (int) (g / d);
            const int64_t r = g % d;
            buffer_offset = (int) (r < local_idx[i] ? r : local_idx[i]);
            const int64_t rest = local_shape[i] - (local_idx[i] - buffer_offset);
            buffer_dim = (int) (rest < d ? rest : d);
        }
        else
        {
            rank_idx = 0;
            for (int j = 0; j < (int) peer_locale_shape[i]; ++j)
            {
                if ((int) local_idx[i] < rank_limits[rl + j])
                {
                    rank_idx = j;
                    break;
                }
            }
            const int base = rank_idx == 0 ? 0 : rank_limits[rl + rank_idx - 1];
            buffer_offset = (int) local_idx[i] - base;
            buffer_dim = rank_limits[rl + rank_idx] - base;
        }
        rank += rank_idx * rank_dim_offset;
        rank_dim_offset *= (int) peer_locale_shape[i];
        off += (size_t) buffer_offset * lin;
        lin *= (size_t) buffer_dim;
        rl += (int) peer_locale_shape[i];
    }
    *dst_rank = rank;
    *dst_offset = off;
}

/*
 * Generic per-element pack (is_pack = 1) or unpack (0) of the shuffler.
 * Follows pack_kernel / unpack_kernel2, legacy/src/tensor/shuffle_mpi_cuda.cu:114-176,
 * 251-300 (CPU twins: shuffle_mpi.hpp:688-706,851-872): elements are visited
 * in natural order of the local shape; the tensor side is addressed through
 * `strides` (get_strided_offset, shuffle_mpi_cuda.cu:100-112), which for a
 * halo-free tensor equals the natural offset.  Elements are opaque
 * `elem_size`-byte values.  Single-threaded like the reference's CPU pack when
 * parallel == 0; with parallel != 0 the outermost dimension is spread over
 * OpenMP threads (used only for the timed CPU baseline).
 */
void orc_shuffle_pack_or_unpack(void* tensor, int nd, int elem_size, const int64_t* local_shape,
                                const int64_t* strides, const int64_t* peer_locale_shape,
                                const int32_t* rank_limits, void* buf, const int32_t* displs,
                                int is_pack, int parallel)
{
    size_t size = 1;
    for (int i = 0; i < nd; ++i)
        size *= (size_t) local_shape[i];
    if (size == 0)
        return;
    char* tp = (char*) tensor;
    char* bp = (char*) buf;
#pragma omp parallel for schedule(static) if (parallel)
    for (long long o = 0; o < (long long) size; ++o)
    {
        int64_t idx[ORC_MAX_DIMS];
        size_t rem = (size_t) o, toff = 0;
        for (int i = 0; i < nd; ++i)
        {
            idx[i] = (int64_t) (rem % (size_t) local_shape[i]);
            rem /= (size_t) local_shape[i];
            toff += (size_t) idx[i] * (size_t) strides[i];
        }
        int rank;
        size_t poff;
        find_destination(nd, idx, local_shape, peer_locale_shape, rank_limits, &rank, &poff);
        char* t = tp + toff * (size_t) elem_size;
        char* b = bp + ((size_t) displs[rank] + poff) * (size_t) elem_size;
        if (is_pack)
            memcpy(b, t, (size_t) elem_size);
        else
            memcpy(t, b, (size_t) elem_size);
    }
}

/*
 * Row-copy pack for 4-D tensors, the structure of the reference's CPU fast
 * path for a sample-parallel source and a spatially decomposed destination
 * (pack_sample_to_spatial4, legacy/include/distconv/tensor/shuffle_mpi.hpp:708-770):
 * OpenMP over the outer loops, every (h, c, n) row of the source cut at the
 * destination's W boundaries and each piece copied with memcpy.  The
 * reference's version assumes equal destination shards; this one cuts at
 * rank_limits, so it equals orc_shuffle_pack_or_unpack (is_pack = 1) on the
 * same tables for uneven splits too (checked in the tests).  Used only by the
 * timed CPU baseline.
 */
void orc_shuffle_pack_rows4(const void* tensor, int elem_size, const int64_t* local_shape,
                            const int64_t* peer_locale_shape, const int32_t* rank_limits,
                            void* buf, const int32_t* displs)
{
    const int64_t W = local_shape[0], H = local_shape[1], C = local_shape[2], N = local_shape[3];
    const int pw = (int) peer_locale_shape[0], ph = (int) peer_locale_shape[1];
    const int32_t* lim_w = rank_limits;
    const int32_t* lim_h = rank_limits + pw;
    const int32_t* lim_c = lim_h + ph;
    const int32_t* lim_n = lim_c + (int) peer_locale_shape[2];
    const char* tp = (const char*) tensor;
    char* bp = (char*) buf;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t n = 0; n < N; ++n)
    {
        for (int64_t c = 0; c < C; ++c)
        {
            int jc = 0, jn = 0;
            while (c >= lim_c[jc]) ++jc;
            while (n >= lim_n[jn]) ++jn;
            const int64_t c0 = jc ? lim_c[jc - 1] : 0, n0 = jn ? lim_n[jn - 1] : 0;
            const int64_t ec = lim_c[jc] - c0;
            for (int64_t h = 0; h < H; ++h)
            {
                int jh = 0;
                while (h >= lim_h[jh]) ++jh;
                const int64_t h0 = jh ? lim_h[jh - 1] : 0;
                const int64_t eh = lim_h[jh] - h0;
                int64_t w0 = 0;
                for (int jw = 0; jw < pw; ++jw)
                {
                    const int64_t ew = lim_w[jw] - w0;
                    if (ew > 0)
                    {
                        const int rank = jw + pw * (jh + ph * (jc + (int) peer_locale_shape[2] * jn));
                        const size_t poff =
                            (size_t) (((n - n0) * ec + (c - c0)) * eh + (h - h0)) * (size_t) ew;
                        const size_t toff = (size_t) (((n * C + c) * H + h) * W + w0);
                        memcpy(bp + ((size_t) displs[rank] + poff) * (size_t) elem_size,
                               tp + toff * (size_t) elem_size, (size_t) ew * (size_t) elem_size);
                    }
                    w0 = lim_w[jw];
                }
            }
        }
    }
}

/*
 * Row-copy pack (is_pack = 1) or unpack (0) for tensors of any rank up to
 * ORC_MAX_DIMS: the structure shared by the reference's CPU fast paths
 * pack_sample_to_spatial4 / 5 (legacy/include/distconv/tensor/shuffle_mpi.hpp:708-849),
 * unpack_sample_to_spatial (:874-879, one memcpy when nothing is cut) and
 * unpack_sample_to_spatial_halo4 / 5 (:881-947): OpenMP over all outer
 * indices, every innermost row cut at the peer grid's limits along dimension
 * 0 and each piece moved with memcpy; the tensor side is addressed through
 * `strides`, so a haloed destination works as in the _halo variants.  (The
 * reference's _halo5 declares its stride array with four entries and indexes
 * it with five, :919-941; the evident five-dimensional loop is restated.)
 * Cuts follow rank_limits, so uneven splits equal orc_shuffle_pack_or_unpack
 * on the same tables (checked in the tests).
 */
void orc_shuffle_rows(void* tensor, int nd, int elem_size, const int64_t* local_shape,
                      const int64_t* strides, const int64_t* peer_locale_shape,
                      const int32_t* rank_limits, void* buf, const int32_t* displs, int is_pack)
{
    size_t outer = 1;
    for (int i = 1; i < nd; ++i)
        outer *= (size_t) local_shape[i];
    if (outer == 0 || local_shape[0] == 0)
        return;
    const int32_t* lim[ORC_MAX_DIMS];
    int rl = 0;
    for (int i = 0; i < nd; ++i)
    {
        lim[i] = rank_limits + rl;
        rl += (int) peer_locale_shape[i];
    }
    char* tp = (char*) tensor;
    char* bp = (char*) buf;
#pragma omp parallel for schedule(static)
    for (long long o = 0; o < (long long) outer; ++o)
    {
        /* outer index -> (i1 .. i_{nd-1}); peer slab and offset inside it per dimension */
        size_t rem = (size_t) o, toff = 0;
        int64_t rank_outer = 0, rank_stride = peer_locale_shape[0];
        int64_t in_slab[ORC_MAX_DIMS], slab_extent[ORC_MAX_DIMS];
        for (int i = 1; i < nd; ++i)
        {
            const int64_t idx = (int64_t) (rem % (size_t) local_shape[i]);
            rem /= (size_t) local_shape[i];
            toff += (size_t) idx * (size_t) strides[i];
            int j = 0;
            while (idx >= lim[i][j])
                ++j;
            const int64_t base = j ? lim[i][j - 1] : 0;
            in_slab[i] = idx - base;
            slab_extent[i] = lim[i][j] - base;
            rank_outer += j * rank_stride;
            rank_stride *= peer_locale_shape[i];
        }
        int64_t w0 = 0;
        for (int jw = 0; jw < (int) peer_locale_shape[0]; ++jw)
        {
            const int64_t ew = lim[0][jw] - w0;
            if (ew > 0)
            {
                /* natural order of the intersection box: dimension 0 fastest */
                size_t poff = 0, lin = (size_t) ew;
                for (int i = 1; i < nd; ++i)
                {
                    poff += (size_t) in_slab[i] * lin;
                    lin *= (size_t) slab_extent[i];
                }
                char* t = tp + (toff + (size_t) w0 * (size_t) strides[0]) * (size_t) elem_size;
                char* b = bp + ((size_t) displs[jw + rank_outer] + poff) * (size_t) elem_size;
                if (is_pack)
                    memcpy(b, t, (size_t) ew * (size_t) elem_size);
                else
                    memcpy(t, b, (size_t) ew * (size_t) elem_size);
            }
            w0 = lim[0][jw];
        }
    }
}
