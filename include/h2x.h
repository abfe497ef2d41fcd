/*
 * h2x.h -- C ABI of the MI355X (gfx950) implementation of DistConv's
 * data-parallel, non-convolution hot path: channel-wise batch-norm statistics
 * (forward and backward), halo pack/unpack of spatially decomposed tensors,
 * channel softmax (forward and backward) and the tensor-shuffler pack/unpack.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream, is
 * asynchronous on that stream, performs no device synchronisation and no
 * allocation unless stated, and returns 0 on success, a positive hipError_t
 * value when the HIP runtime reported an error, or a negative h2x_status.
 * The library never aborts the process.
 *
 * Conventions shared with the reference (paths relative to the reference
 * checkout):
 *   - dimension order is innermost first: an "NCHW" tensor has shape
 *     {W, H, C, N}; channel is dimension nd-2, sample is nd-1
 *     (legacy/include/distconv/distconv.hpp:103-109);
 *   - "real" shape = local shape + 2 * halo width per dimension
 *     (legacy/include/distconv/tensor/tensor_mpi.hpp:497-498);
 *   - LHS = 0, RHS = 1 (legacy/include/distconv/base.hpp:23).
 */
#ifndef H2X_H_INCLUDED
#define H2X_H_INCLUDED

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define H2X_MAX_DIMS 6

/** A hipStream_t passed through an opaque pointer (NULL = the null stream). */
typedef void* h2x_stream_t;

typedef enum h2x_status
{
    H2X_SUCCESS = 0,
    H2X_ERR_INVALID_ARGUMENT = -1,
    H2X_ERR_UNSUPPORTED = -2,
    H2X_ERR_TOO_LARGE = -3,
    H2X_ERR_SCRATCH_LIMIT = -4 /* beyond the fixed capacity of an entry point that allocates nothing */
} h2x_status;

/** Element type of floating-point tensors (batch-norm, softmax, halo accumulate). */
typedef enum h2x_dtype
{
    H2X_F32 = 0,
    H2X_F64 = 1
} h2x_dtype;

/** legacy/include/distconv/base.hpp:23 */
typedef enum h2x_side
{
    H2X_LHS = 0,
    H2X_RHS = 1
} h2x_side;

/** legacy/include/distconv/tensor/halo_exchange.hpp:8-9 */
typedef enum h2x_halo_op
{
    H2X_HALO_ID = 0,
    H2X_HALO_SUM = 1,
    H2X_HALO_MAX = 2,
    H2X_HALO_MIN = 3
} h2x_halo_op;

/* ------------------------------------------------------------------------ */
/* Library                                                                   */
/* ------------------------------------------------------------------------ */

/** ABI version of this header; bumped on any incompatible change. */
int h2x_abi_version(void);

/** Human-readable text for a value returned by any h2x_* function. */
const char* h2x_status_string(int status);

/* ------------------------------------------------------------------------ */
/* Batch normalisation                                                       */
/*                                                                           */
/* Tensor geometry of x, y, dy, dx: element (n, c, i) of the local tensor    */
/* lives at base[(n * num_channels + c) * spatial_real_size + i] for         */
/* 0 <= i < spatial_size.  spatial_size is the product of the local spatial  */
/* extents, spatial_real_size the same product over the real (haloed)        */
/* extents; they differ only when the outermost spatial dimension carries a  */
/* halo, and `base` then is the tensor's get_base_ptr().  This is the        */
/* geometry the reference's optimised kernels accept                         */
/* (legacy/src/dnn_backend/batchnorm.cu:134-190,210-230).                    */
/* Per-channel vectors (sums, mean, var, scale, ...) are dense arrays of     */
/* num_channels elements.                                                    */
/* ------------------------------------------------------------------------ */

/**
 * Bytes of device workspace the two reduction entry points need for
 * `num_channels` channels.  The workspace holds fp64 partial sums, one set per
 * workgroup; it needs no initialisation and keeps no state between calls.  One
 * workspace must not be used by two calls that may run concurrently.
 */
size_t h2x_bn_workspace_bytes(int num_channels);

/**
 * sums[c] = sum over (n, i) of x; sqsums[c] = sum of x*x.
 * Replaces batchnorm::channel_sums_and_sqsums
 * (legacy/include/distconv/dnn_backend/batchnorm.hpp:22-28,
 *  legacy/src/dnn_backend/batchnorm.cu:192-271).  Outputs are overwritten
 * (the reference zeroes them and accumulates with atomics); with
 * num_samples == 0 or spatial_size == 0 they are set to zero.  Accumulation
 * is in fp64 with a fixed reduction order, so results are run-to-run
 * deterministic.
 */
int h2x_bn_channel_sums_and_sqsums(h2x_dtype dtype,
                                   int num_samples,
                                   int num_channels,
                                   size_t spatial_size,
                                   size_t spatial_real_size,
                                   const void* x,
                                   void* sums,
                                   void* sqsums,
                                   void* workspace,
                                   h2x_stream_t stream);

/**
 * h2x_bn_channel_sums_and_sqsums for callers that cannot allocate device
 * memory and have no workspace to pass: code under HIP graph capture, serving
 * loops, harnesses that forbid allocation.  It has no counterpart in the
 * reference.  Same arguments, kernels and results (bit for bit) as
 * h2x_bn_channel_sums_and_sqsums, but the partial sums live in a 1 MiB array
 * inside the library's device image, one copy per device; the call performs no
 * allocation of any kind.  num_channels above h2x_bn_static_max_channels() is
 * rejected with H2X_ERR_SCRATCH_LIMIT.  All calls on one device share that array:
 * two calls that may run concurrently on one device (different streams) race.
 * The array's device address is looked up on the first call on each device
 * (hipGetSymbolAddress, no allocation); make that call outside graph capture.
 */
int h2x_bn_channel_sums_and_sqsums_static(h2x_dtype dtype,
                                          int num_samples,
                                          int num_channels,
                                          size_t spatial_size,
                                          size_t spatial_real_size,
                                          const void* x,
                                          void* sums,
                                          void* sqsums,
                                          h2x_stream_t stream);

/** Largest num_channels h2x_bn_channel_sums_and_sqsums_static accepts. */
size_t h2x_bn_static_max_channels(void);

/**
 * In place: mean = sums / n; var = max(sqsums / n - mean^2, 0) * n / (n - 1);
 * running_x = decay * running_x + (1 - decay) * x.  With num_per_sum == 0
 * only var is written (set to 1).  Replaces batchnorm::sums_to_statistics
 * (batchnorm.hpp:30-37, batchnorm.cu:288-346).
 */
int h2x_bn_sums_to_statistics(h2x_dtype dtype,
                              int num_channels,
                              size_t num_per_sum,
                              double decay,
                              void* mean_inout,
                              void* var_inout,
                              void* running_mean,
                              void* running_var,
                              h2x_stream_t stream);

/**
 * y = (x - mean) * rsqrt(var + epsilon) * scale + bias.
 * Replaces batchnorm::batch_normalization (batchnorm.hpp:39-49,
 * batchnorm.cu:420-573).  x and y have their own real sizes.
 */
int h2x_bn_batch_normalization(h2x_dtype dtype,
                               int num_samples,
                               int num_channels,
                               size_t spatial_size,
                               size_t x_spatial_real_size,
                               size_t y_spatial_real_size,
                               const void* x,
                               const void* mean,
                               const void* var,
                               const void* scale,
                               const void* bias,
                               void* y,
                               double epsilon,
                               h2x_stream_t stream);

/**
 * Backward reductions per channel (r = rsqrt(var + epsilon)):
 *   dscale = sum dy * (x - mean) * r;   dbias = sum dy;
 *   dmean  = - sum dy * scale * r;
 *   dvar   = - sum dy * scale * (x - mean) * r^3 / 2.
 * Replaces batchnorm::backprop1 (batchnorm.hpp:68-81, batchnorm.cu:982-1230).
 * Outputs are overwritten; fp64 accumulation, deterministic.
 */
int h2x_bn_backprop1(h2x_dtype dtype,
                     int num_samples,
                     int num_channels,
                     size_t spatial_size,
                     size_t x_spatial_real_size,
                     size_t dy_spatial_real_size,
                     const void* x,
                     const void* dy,
                     const void* mean,
                     const void* var,
                     const void* scale,
                     void* dscale,
                     void* dbias,
                     void* dmean,
                     void* dvar,
                     double epsilon,
                     void* workspace,
                     h2x_stream_t stream);

/**
 * dx = dy * scale * r + dmean / n + dvar * 2 / (n - 1) * (x - mean), with
 * n = num_per_sum.  dx may be x itself (the same elements at the same
 * addresses, batchnorm.cu:1303-1314); buffers that overlap in any other way
 * are not supported.  Replaces batchnorm::backprop2
 * (batchnorm.hpp:83-96, batchnorm.cu:1371-1559).
 */
int h2x_bn_backprop2(h2x_dtype dtype,
                     int num_samples,
                     int num_channels,
                     size_t spatial_size,
                     size_t x_spatial_real_size,
                     size_t dy_spatial_real_size,
                     size_t dx_spatial_real_size,
                     size_t num_per_sum,
                     const void* x,
                     const void* dy,
                     const void* mean,
                     const void* var,
                     const void* scale,
                     const void* dmean,
                     const void* dvar,
                     void* dx,
                     double epsilon,
                     h2x_stream_t stream);

/**
 * Forward pass of a rank whose statistics are its own (one rank, or
 * global_stats == false: no all-reduce between the stages): what
 *   h2x_bn_channel_sums_and_sqsums, h2x_bn_sums_to_statistics(num_per_sum, decay)
 *   and h2x_bn_batch_normalization
 * leave in mean, var, running_mean, running_var and y, bit for bit, in two
 * launches instead of four: the normalising kernel finishes the sums itself.
 * This is BatchNormalization::forward without its allreduce stage
 * (legacy/include/distconv/dnn_backend/batchnorm.hpp:171-250); the staged entry
 * points remain for ranks that all-reduce between stage 1 and stage 2.
 */
int h2x_bn_forward_local(h2x_dtype dtype,
                         int num_samples,
                         int num_channels,
                         size_t spatial_size,
                         size_t x_spatial_real_size,
                         size_t y_spatial_real_size,
                         const void* x,
                         const void* scale,
                         const void* bias,
                         size_t num_per_sum,
                         double decay,
                         double epsilon,
                         void* mean,
                         void* var,
                         void* running_mean,
                         void* running_var,
                         void* y,
                         void* workspace,
                         h2x_stream_t stream);

/**
 * Backward pass likewise: h2x_bn_backprop1 followed by h2x_bn_backprop2 with
 * the sums it produced, bit for bit, in two launches instead of three
 * (BatchNormalization::backward without its allreduce stage,
 * batchnorm.hpp:360-475).  dx may be x itself.
 */
int h2x_bn_backward_local(h2x_dtype dtype,
                          int num_samples,
                          int num_channels,
                          size_t spatial_size,
                          size_t x_spatial_real_size,
                          size_t dy_spatial_real_size,
                          size_t dx_spatial_real_size,
                          size_t num_per_sum,
                          const void* x,
                          const void* dy,
                          const void* mean,
                          const void* var,
                          const void* scale,
                          void* dscale,
                          void* dbias,
                          void* dmean,
                          void* dvar,
                          void* dx,
                          double epsilon,
                          void* workspace,
                          h2x_stream_t stream);

/**
 * Local part of a tensor given by shape and strides, for tensors that carry a
 * halo on an inner spatial dimension.  Innermost first; the last two
 * dimensions are channel and sample; num_dims is 3, 4 or 5.  strides are in
 * elements of the real (haloed) allocation (Tensor::get_strides(),
 * legacy/include/distconv/tensor/tensor.hpp:291-298) and strides[0] must be 1;
 * the data pointer that goes with it is the tensor's get_base_ptr().
 */
/* (The transform and sum entry points further down accept any 1 to
 * H2X_MAX_DIMS dimensions and any strides.) */
typedef struct h2x_tensor_geometry
{
    int32_t num_dims;
    int32_t reserved;
    int64_t local_shape[H2X_MAX_DIMS];
    int64_t strides[H2X_MAX_DIMS];
} h2x_tensor_geometry;

/**
 * The four tensor passes for arbitrarily haloed tensors: what the reference's
 * generic kernels cover (legacy/src/dnn_backend/batchnorm.cu:39-90, 369-418,
 * 899-980, 1303-1369, chosen by its drivers at :210-248, 514-573, 1168-1230,
 * 1503-1559).  Same results as the dense entry points on the same elements;
 * a geometry that is dense inside its segments is forwarded to them.
 * local_shape[num_dims - 1] must equal num_samples.
 */
int h2x_bn_channel_sums_and_sqsums_strided(h2x_dtype dtype,
                                           int num_samples,
                                           const h2x_tensor_geometry* x_geometry,
                                           const void* x,
                                           void* sums,
                                           void* sqsums,
                                           void* workspace,
                                           h2x_stream_t stream);

int h2x_bn_batch_normalization_strided(h2x_dtype dtype,
                                       int num_samples,
                                       const h2x_tensor_geometry* x_geometry,
                                       const h2x_tensor_geometry* y_geometry,
                                       const void* x,
                                       const void* mean,
                                       const void* var,
                                       const void* scale,
                                       const void* bias,
                                       void* y,
                                       double epsilon,
                                       h2x_stream_t stream);

int h2x_bn_backprop1_strided(h2x_dtype dtype,
                             int num_samples,
                             const h2x_tensor_geometry* x_geometry,
                             const h2x_tensor_geometry* dy_geometry,
                             const void* x,
                             const void* dy,
                             const void* mean,
                             const void* var,
                             const void* scale,
                             void* dscale,
                             void* dbias,
                             void* dmean,
                             void* dvar,
                             double epsilon,
                             void* workspace,
                             h2x_stream_t stream);

int h2x_bn_backprop2_strided(h2x_dtype dtype,
                             int num_samples,
                             size_t num_per_sum,
                             const h2x_tensor_geometry* x_geometry,
                             const h2x_tensor_geometry* dy_geometry,
                             const h2x_tensor_geometry* dx_geometry,
                             const void* x,
                             const void* dy,
                             const void* mean,
                             const void* var,
                             const void* scale,
                             const void* dmean,
                             const void* dvar,
                             void* dx,
                             double epsilon,
                             h2x_stream_t stream);

/**
 * h2x_bn_forward_local and h2x_bn_backward_local for tensors given by shape
 * and strides (haloed shards): the same two launches, the same bits as the
 * staged _strided calls.  Where the tensors of a call take different families
 * of kernels (a haloed tensor with short segments beside a dense one), the
 * staged calls run instead, with the same results.
 */
int h2x_bn_forward_local_strided(h2x_dtype dtype,
                                 int num_samples,
                                 const h2x_tensor_geometry* x_geometry,
                                 const h2x_tensor_geometry* y_geometry,
                                 const void* x,
                                 const void* scale,
                                 const void* bias,
                                 size_t num_per_sum,
                                 double decay,
                                 double epsilon,
                                 void* mean,
                                 void* var,
                                 void* running_mean,
                                 void* running_var,
                                 void* y,
                                 void* workspace,
                                 h2x_stream_t stream);
int h2x_bn_backward_local_strided(h2x_dtype dtype,
                                  int num_samples,
                                  size_t num_per_sum,
                                  const h2x_tensor_geometry* x_geometry,
                                  const h2x_tensor_geometry* dy_geometry,
                                  const h2x_tensor_geometry* dx_geometry,
                                  const void* x,
                                  const void* dy,
                                  const void* mean,
                                  const void* var,
                                  const void* scale,
                                  void* dscale,
                                  void* dbias,
                                  void* dmean,
                                  void* dvar,
                                  void* dx,
                                  double epsilon,
                                  void* workspace,
                                  h2x_stream_t stream);

/**
 * The local part of a haloed tensor as it lies in memory: the real (allocated)
 * extents and where the interior starts in them.  Innermost first; the last
 * two dimensions are channel and sample and carry no halo; num_dims is 3, 4
 * or 5 (Tensor::get_local_shape(), get_local_real_shape() and the halo width
 * of each dimension, legacy/include/distconv/tensor/tensor_base.hpp:344-361).
 */
typedef struct h2x_haloed_geometry
{
    int32_t num_dims;
    int32_t reserved;
    int64_t local_shape[H2X_MAX_DIMS];
    int64_t real_shape[H2X_MAX_DIMS];
    int64_t lower_halo[H2X_MAX_DIMS]; /* real index of the first interior element */
} h2x_haloed_geometry;

/**
 * Normalise and input gradient for tensors that all have the geometry given
 * (x and y; x, dy and dx), leaving the halo of the OUTPUT cleared: the result
 * of h2x_bn_batch_normalization_strided (h2x_bn_backprop2_strided) followed by
 * h2x_halo_clear on every spatial dimension of the output, bit for bit, in one
 * pass over the real tensors.  No counterpart in the reference, whose
 * Convolution::forward clears the halos of its input before every exchange
 * (legacy/include/distconv/dnn_backend/convolution.hpp:400-411): a layer that
 * feeds a convolution can hand over its output with the halo already cleared.
 * The kernels walk the whole allocation in aligned vectors, so the 8-byte gaps
 * between interior rows cost no partial writes (a shard of NCDHW 4 x 64 x 64^3
 * with a halo of 1: forward + backward at 0.76-0.78 of the HBM peak, the rate
 * of the calls that leave the halo alone, without the clear_halo launches that
 * would follow them).  The pointers are the starts of the allocations
 * (Tensor::get_buffer()), not of the interiors.  Halo cells of the inputs are
 * read and ignored; dx_buffer may be x_buffer.  Falls back to single elements
 * when a segment of the real tensor is no multiple of 16 bytes long or a
 * buffer is not 16-byte aligned.
 */
int h2x_bn_batch_normalization_clearing(h2x_dtype dtype,
                                        const h2x_haloed_geometry* geometry,
                                        const void* x_buffer,
                                        const void* mean,
                                        const void* var,
                                        const void* scale,
                                        const void* bias,
                                        void* y_buffer,
                                        double epsilon,
                                        h2x_stream_t stream);
int h2x_bn_backprop2_clearing(h2x_dtype dtype,
                              size_t num_per_sum,
                              const h2x_haloed_geometry* geometry,
                              const void* x_buffer,
                              const void* dy_buffer,
                              const void* mean,
                              const void* var,
                              const void* scale,
                              const void* dmean,
                              const void* dvar,
                              void* dx_buffer,
                              double epsilon,
                              h2x_stream_t stream);

/**
 * Launch audit, on the host: no GPU call is made and no pointer is followed.
 * No counterpart in the reference, whose kernels check nothing of the kind;
 * it exists so that the choice of kernels and their indexing can be verified
 * on a machine without a GPU.  The entry point named by `stage` plans its
 * launches for tensors of the given geometries (x; y or dy; dx - as many as
 * the stage takes) at the given base addresses (only their alignment and
 * whether x and dx share memory matter), and every workgroup and lane of
 * every planned launch is then played on the CPU through the index maps the
 * kernels use.  Per launch and tensor the report says how many elements are
 * loaded and stored, how many of those accesses fall outside the interior
 * elements of the tensor (`outside`: must be 0; halo cells and anything beyond
 * the allocation count), how many interior elements no lane owns (`missed`:
 * must be 0) and how many are owned by more than one (`owned_twice`: must be
 * 0; a reduction would add them twice).  Owning an element means adding it
 * into a sum or storing its result; elements that two overlapping vectors
 * share are loaded, and where allowed stored, by both but owned by one.
 * The two-launch stages go through h2x_bn_forward_local / _backward_local for
 * geometries of three dimensions {spatial, channels, samples} with strides
 * {1, real, real * channels}, through their _strided twins otherwise.  Returns what the entry point returns; H2X_ERR_TOO_LARGE if it
 * plans more than H2X_BN_AUDIT_MAX_LAUNCHES launches.  Cost: proportional to
 * the elements of the tensors; meant for tests.
 */
typedef enum h2x_bn_stage
{
    H2X_BN_STAGE_SUMS = 0,          /* h2x_bn_channel_sums_and_sqsums_strided */
    H2X_BN_STAGE_NORMALIZE = 1,     /* h2x_bn_batch_normalization_strided */
    H2X_BN_STAGE_BACKPROP1 = 2,     /* h2x_bn_backprop1_strided */
    H2X_BN_STAGE_BACKPROP2 = 3,     /* h2x_bn_backprop2_strided */
    H2X_BN_STAGE_FORWARD_LOCAL = 4, /* h2x_bn_forward_local(_strided) */
    H2X_BN_STAGE_BACKWARD_LOCAL = 5 /* h2x_bn_backward_local(_strided) */
} h2x_bn_stage;

#define H2X_BN_AUDIT_MAX_LAUNCHES 8

typedef struct h2x_bn_audit_tensor
{
    uint64_t loads, stores; /* elements */
    uint64_t outside, missed, owned_twice;
} h2x_bn_audit_tensor;

typedef struct h2x_bn_audit_launch
{
    int32_t kernel; /* 0 sums, 1 normalise, 2 backprop1, 3 backprop2, 4 finish, 5 statistics, 6 fill, 7 halo-clearing */
    int32_t family; /* 0 dense, 1 strided (padded rows, folded samples), 2 short segments */
    int32_t vector_width; /* elements per access */
    int32_t tail;         /* short family: 0 whole vectors, 1 overlapping last vector, 2 element by element */
    int32_t folded;       /* samples folded into the rows of one segment */
    int32_t fused;        /* finishes the preceding reduction itself */
    uint32_t grid_x, grid_y;
    uint64_t partials_bytes;    /* reductions: bytes of partial sums the launch can write in the workspace */
    uint64_t partials_capacity; /* reductions: bytes the library reserves for them */
    int32_t num_tensors;
    int32_t reserved;
    h2x_bn_audit_tensor tensor[3];
} h2x_bn_audit_launch;

typedef struct h2x_bn_audit_report
{
    int32_t num_launches;
    int32_t reserved;
    uint64_t workspace_bytes; /* h2x_bn_workspace_bytes of the channel count */
    h2x_bn_audit_launch launch[H2X_BN_AUDIT_MAX_LAUNCHES];
} h2x_bn_audit_report;

int h2x_bn_audit(h2x_bn_stage stage,
                 h2x_dtype dtype,
                 int num_samples,
                 const h2x_tensor_geometry* const* geometry,
                 const uint64_t* address,
                 h2x_bn_audit_report* report);

/**
 * The same audit for h2x_bn_batch_normalization_clearing (`backward` 0: tensors
 * x, y) and h2x_bn_backprop2_clearing (`backward` 1: x, dy, dx), which walk the
 * real local tensor.  Addresses are the allocation starts.  Per tensor:
 * `outside` counts accesses beyond the real tensor and, for the output, cells
 * the kernel's interior test places on the wrong side (a halo cell computed or
 * an interior cell zeroed; the interior is enumerated independently from the
 * local shape and the halo widths); `missed` / `owned_twice` count real cells
 * of the output that are stored never / more than once.  All must be 0.  The
 * launch is reported with kernel 7.
 */
int h2x_bn_audit_clearing(int backward,
                          h2x_dtype dtype,
                          const h2x_haloed_geometry* geometry,
                          const uint64_t* address,
                          h2x_bn_audit_report* report);

/**
 * Launch audit of the copy entry points (halo pack / unpack / clear / fused
 * exchange, shuffle plans, pack and unpack), on the host: no GPU call is made
 * and no pointer is followed.  No counterpart in the reference.  Between
 * h2x_copy_audit_begin and h2x_copy_audit_end the calling thread's calls to
 * those entry points plan their launches as usual, and every launch is played
 * on the CPU, workgroup by workgroup and lane by lane, through the code of the
 * kernel itself with memory accesses counted instead of made.  The caller
 * registers the address ranges of its tensors and buffers (any addresses: real
 * host allocations serve as well as imaginary ones) and, per
 * range, two arrays of one counter per byte: `loads[i]` / `stores[i]` say how
 * often byte base + i would be loaded / stored (saturating at 255; either may
 * be null).  What falls outside every range is counted in the report
 * (`outside_loads`, `outside_stores`, in bytes: must be 0), as are accesses not
 * aligned as their instruction needs (`misaligned`: must be 0).  A shuffle plan
 * made while an audit is open serves audited launches only; destroy it as any
 * other.  Cost: proportional to the elements moved; meant for tests on machines
 * without a GPU.  The stream argument of the audited calls is ignored.
 */
typedef struct h2x_copy_audit_region
{
    uint64_t base;
    uint64_t bytes;
    uint8_t* loads;
    uint8_t* stores;
} h2x_copy_audit_region;

typedef struct h2x_copy_audit_report
{
    uint64_t launches;
    uint64_t workgroups;
    uint64_t outside_loads, outside_stores; /* bytes */
    uint64_t misaligned;                    /* accesses */
} h2x_copy_audit_report;

int h2x_copy_audit_begin(void);
/** Registers one address range with the open audit (the counter arrays must outlive it). */
int h2x_copy_audit_add_region(const h2x_copy_audit_region* region);
/** Closes the audit of the calling thread and reports (report may be null). */
int h2x_copy_audit_end(h2x_copy_audit_report* report);

/* ------------------------------------------------------------------------ */
/* Elementwise transforms and sums over dimensions                           */
/* ------------------------------------------------------------------------ */

/**
 * The operations tensor::Transform is instantiated with on this path
 * (legacy/include/distconv/tensor/algorithms/transform_cuda.hpp:359-693).  The
 * reference compiles a kernel per functor; here they are named.
 */
typedef enum h2x_transform_op
{
    /** 1 tensor: x = x * params[0] (internal::ScaleFunctor, legacy/src/tensor/tensor_mpi_cuda.cu:86-98). */
    H2X_TRANSFORM_SCALE = 0,
    /** 2 tensors: t1 = t0. */
    H2X_TRANSFORM_COPY = 1,
    /** 2 tensors: t1 = params[0] * t0 + params[1] (CastScaleBias with equal types, tensor_mpi_cuda.cu:113-135). */
    H2X_TRANSFORM_SCALE_BIAS = 2,
    /** 4 tensors (sums -> mean, sqsums -> var, running_mean, running_var), in place, with
     *  params[0] = num_per_sum, params[1] = decay: what h2x_bn_sums_to_statistics computes,
     *  expressed as the four-tensor transform the reference uses
     *  (legacy/src/dnn_backend/batchnorm.cu:288-346). */
    H2X_TRANSFORM_SUMS_TO_STATISTICS = 3
} h2x_transform_op;

/**
 * Applies `op` to corresponding elements of the local parts (interiors) of
 * `num_tensors` tensors.  Each tensor comes with its own geometry: all local
 * shapes must be equal, strides are each tensor's own (halos), the pointers
 * are the tensors' get_base_ptr().  Here a geometry may have 1 to
 * H2X_MAX_DIMS dimensions of any meaning and any strides.  `params` holds
 * four doubles (may be NULL for COPY).  Replaces tensor::Transform
 * (transform_cuda.hpp:359-693) for the named operations.
 */
int h2x_tensor_transform(h2x_transform_op op,
                         h2x_dtype dtype,
                         int num_tensors,
                         const h2x_tensor_geometry* const* geometries,
                         void* const* tensors,
                         const double* params,
                         h2x_stream_t stream);

/** Bytes of device workspace h2x_tensor_reduce_sum needs for this pair of geometries (fp64 partial sums, no initialisation). */
size_t h2x_tensor_reduce_sum_workspace_bytes(const h2x_tensor_geometry* src_geometry,
                                             const h2x_tensor_geometry* dst_geometry);

/**
 * dst += sum of src (or of src * src when `square` is set) over every
 * dimension in which dst has extent 1 and src has more.  Each local extent of
 * dst must be 1 or equal to src's; src's local_shape is the region summed
 * (the reference's local_reduction_shape).  As in the reference the
 * destination is accumulated into, so it is zeroed by the caller first
 * (tensor::ReduceSum and TransformReduceSum,
 * legacy/include/distconv/tensor/algorithms/reduce_sum_cuda.hpp:56-113,388-439;
 * the all-reduce over ranks that follows there is the caller's).  fp64
 * accumulation in a fixed order: deterministic.
 */
int h2x_tensor_reduce_sum(h2x_dtype dtype,
                          const h2x_tensor_geometry* src_geometry,
                          const void* src,
                          const h2x_tensor_geometry* dst_geometry,
                          void* dst,
                          int square,
                          void* workspace,
                          h2x_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Channel softmax: dense [num_samples][num_channels][spatial_size] tensors,  */
/* softmax taken over the channel dimension.                                  */
/* ------------------------------------------------------------------------ */

/**
 * m = max(FLT_MIN, max_c x); e = exp(x - m); y = max(e * (1 / sum_c e), FLT_MIN)
 * (DBL_MIN for f64).  Replaces Softmax::forward in SoftmaxMode::CHANNEL
 * (legacy/src/dnn_backend/softmax.cu:538-619,705-747).
 */
int h2x_softmax_channel_forward(h2x_dtype dtype,
                                int num_samples,
                                int num_channels,
                                size_t spatial_size,
                                const void* x,
                                void* y,
                                h2x_stream_t stream);

/**
 * dp = sum_c y * dy; dx = y > FLT_MIN ? y * (dy - dp) : 0.
 * Replaces Softmax::backward in SoftmaxMode::CHANNEL
 * (legacy/src/dnn_backend/softmax.cu:621-701,749-768).
 */
int h2x_softmax_channel_backward(h2x_dtype dtype,
                                 int num_samples,
                                 int num_channels,
                                 size_t spatial_size,
                                 const void* y,
                                 const void* dy,
                                 void* dx,
                                 h2x_stream_t stream);

/* Instance mode: softmax over all elements of a sample (dense tensors, a      */
/* sample is `sample_size` contiguous elements).  The reference runs it as     */
/* three forward and two backward stages with an all-reduce of the per-sample  */
/* scalars between them when a sample is spread over ranks                     */
/* (legacy/src/dnn_backend/softmax.cu:705-784,                                */
/*  legacy/include/distconv/dnn_backend/softmax.hpp:52-62); the stages are    */
/* the entry points.  Per-sample vectors hold num_samples elements.           */

/** Workspace (fp64 partials) of the three reducing stages; no initialisation needed. */
size_t h2x_softmax_instance_workspace_bytes(int num_samples);

/** sample_max[n] = max(min_normal, max_i x): compute_max, softmax.cu:357-381. */
int h2x_softmax_instance_max(h2x_dtype dtype, int num_samples, size_t sample_size, const void* x,
                             void* sample_max, void* workspace, h2x_stream_t stream);

/** y = exp(x - sample_max[n]); sample_exp[n] = sum_i y: compute_exp, softmax.cu:394-421. */
int h2x_softmax_instance_exp(h2x_dtype dtype, int num_samples, size_t sample_size, const void* x,
                             const void* sample_max, void* y, void* sample_exp, void* workspace,
                             h2x_stream_t stream);

/** y = max(y / sample_exp[n], sqrt(min_normal)) in place: compute_softmax, softmax.cu:424-456. */
int h2x_softmax_instance_normalize(h2x_dtype dtype, int num_samples, size_t sample_size,
                                   const void* sample_exp, void* y, h2x_stream_t stream);

/**
 * The three forward stages for samples that are whole on this rank (no
 * all-reduce between them, softmax.hpp:52-62 with one process per sample): what
 * h2x_softmax_instance_max, _exp and _normalize leave in y, sample_max and
 * sample_exp, bit for bit, in four passes over the tensors instead of five: the
 * exponentials are summed without being stored and made again from x when y is
 * written.  The staged entry points remain for samples spread over ranks.
 */
int h2x_softmax_instance_forward_local(h2x_dtype dtype, int num_samples, size_t sample_size,
                                       const void* x, void* y, void* sample_max, void* sample_exp,
                                       void* workspace, h2x_stream_t stream);

/** sample_dp[n] = sum_i y * dy: bp_dotproduct, softmax.cu:458-481. */
int h2x_softmax_instance_dot(h2x_dtype dtype, int num_samples, size_t sample_size, const void* y,
                             const void* dy, void* sample_dp, void* workspace, h2x_stream_t stream);

/** dx = y > sqrt(min_normal) ? y * (dy - sample_dp[n]) : 0: bp_compute_gradient, softmax.cu:483-536. */
int h2x_softmax_instance_gradient(h2x_dtype dtype, int num_samples, size_t sample_size,
                                  const void* y, const void* dy, const void* sample_dp, void* dx,
                                  h2x_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Halo pack / unpack                                                        */
/* ------------------------------------------------------------------------ */

/**
 * One halo strip of one tensor.  `tensor` is the start of the real (haloed)
 * allocation (get_buffer()), `real_shape` its real extents, innermost first.
 * The strip is `width` cells thick along `dim`, spans the full real extent of
 * every other dimension and starts, along `dim`, at
 *   LHS outer: 0              LHS inner: width
 *   RHS outer: shape - width  RHS inner: shape - 2 * width
 * (legacy/include/distconv/tensor/halo_cuda.hpp:59-81).  `buffer` holds the
 * strip in natural (innermost-first) order of the strip's own extents, the
 * layout of the reference's generic traversal (halo_cuda.hpp:53-86).
 * pack:   buffer[o] = tensor[strip(o)]
 * unpack: tensor[strip(o)] = op(tensor[strip(o)], buffer[o])
 * (legacy/include/distconv/tensor/halo_packing_cuda.hpp:60-83).
 */
typedef struct h2x_halo_face
{
    void* tensor;
    void* buffer;
    int64_t real_shape[H2X_MAX_DIMS];
    int32_t num_dims;
    int32_t dim;
    int32_t side;    /* h2x_side */
    int32_t width;
    int32_t inner;   /* 0: outer (halo) strip, 1: inner (boundary) strip */
    int32_t is_pack; /* 1: tensor -> buffer, 0: buffer -> tensor */
    int32_t op;      /* h2x_halo_op, used when unpacking */
    int32_t reserved;
} h2x_halo_face;

/** Number of elements of the strip described by (real_shape, dim, width): legacy/include/distconv/tensor/halo_exchange_cuda.hpp:267-271. */
size_t h2x_halo_size(int num_dims, const int64_t* real_shape, int dim, int width);

/**
 * Pack or unpack one strip.  `inner` follows
 * (is_pack && !is_reverse) || (!is_pack && is_reverse)
 * (halo_packing_cuda.hpp:100); width == 0 is a no-op.  Replaces
 * halo_exchange_cuda::pack_or_unpack<T> (halo_packing_cuda.hpp:143-167,
 * legacy/src/tensor/halo_exchange_cuda.cu:12-40).
 */
int h2x_halo_pack_or_unpack(h2x_dtype dtype,
                            void* tensor,
                            int num_dims,
                            const int64_t* real_shape,
                            int dim,
                            int side,
                            int width,
                            void* buffer,
                            int is_pack,
                            int is_reverse,
                            int op,
                            h2x_stream_t stream);

/**
 * The same for `num_faces` independent strips in as few launches as possible
 * (both sides of a dimension, several tensors).  Faces of one call must not
 * overlap in what they write.  `faces` is host memory, read before return.
 */
int h2x_halo_pack_or_unpack_batched(h2x_dtype dtype,
                                    const h2x_halo_face* faces,
                                    int num_faces,
                                    h2x_stream_t stream);

/**
 * tensor[strip] = 0 for every face of `faces` (tensor, real_shape, num_dims, dim,
 * side, width and inner are read; inner = 0 names the halo strip), any number of
 * tensors, dimensions and sides, in as few launches as the kinds of strips allow
 * (one for the strips of the innermost dimension, one per 16 of the others).
 * What a loop of TensorImplHelper::clear_halo over dimensions and tensors does
 * (legacy/src/tensor/tensor_mpi_cuda.cu:14-84; the loop:
 * legacy/include/distconv/dnn_backend/convolution.hpp:400-411), and its building
 * block where only some sides need clearing: a side whose neighbour will
 * overwrite the whole strip in the exchange that follows need not be cleared.
 * `faces` is host memory, read before return.
 */
int h2x_halo_clear_batched(h2x_dtype dtype,
                           const h2x_halo_face* faces,
                           int num_faces,
                           h2x_stream_t stream);

/**
 * tensor[strip] = 0 for the outer strips of `dim` on both sides, width =
 * the real halo width.  Replaces TensorImplHelper::clear_halo
 * (legacy/src/tensor/tensor_mpi_cuda.cu:14-84).
 */
int h2x_halo_clear(h2x_dtype dtype,
                   void* tensor,
                   int num_dims,
                   const int64_t* real_shape,
                   int dim,
                   int width,
                   h2x_stream_t stream);

/**
 * One strip moved straight from the tensor of one rank into the tensor of its
 * neighbour on the same device: what
 *   h2x_halo_pack_or_unpack(src, ..., dim, src_side, width, buf, is_pack=1, is_reverse, ...)
 * followed by
 *   h2x_halo_pack_or_unpack(dst, ..., dim, opposite side, width, buf, is_pack=0, is_reverse, op)
 * leaves in `dst`, without the buffer.  Forward (is_reverse = 0): the interior
 * strip of `src` at `src_side` lands in the halo of `dst` on the opposite side;
 * reverse: the halo of `src` at `src_side` is combined with `op` into the
 * interior strip of `dst` on the opposite side.  The two real shapes must agree
 * in every dimension but `dim`.  The reference always stages strips through
 * buffers (legacy/include/distconv/tensor/halo_exchange_cuda_mpi.hpp:25-100,
 * halo_packing_cuda.hpp:143-167); this entry point is for neighbours that
 * share a device.
 */
typedef struct h2x_halo_transfer
{
    const void* src;  /* start of the source rank's real allocation */
    void* dst;        /* start of the destination rank's real allocation */
    int64_t src_real_shape[H2X_MAX_DIMS];
    int64_t dst_real_shape[H2X_MAX_DIMS];
    int32_t num_dims;
    int32_t dim;
    int32_t src_side;   /* h2x_side: the side of `src` that faces `dst` */
    int32_t width;
    int32_t is_reverse;
    int32_t op;         /* h2x_halo_op */
} h2x_halo_transfer;

/**
 * `num_transfers` strips in as few launches as possible.  No transfer of a
 * call may write what another one reads or writes (true for all strips of one
 * dimension of an exchange).  `transfers` is host memory, read before return.
 */
int h2x_halo_exchange_fused(h2x_dtype dtype,
                            const h2x_halo_transfer* transfers,
                            int num_transfers,
                            h2x_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Tensor shuffler pack / unpack                                             */
/* ------------------------------------------------------------------------ */

/**
 * Geometry of one rank's side of a shuffle, taken from the tables the
 * reference's shuffler constructor builds
 * (legacy/include/distconv/tensor/shuffle_mpi_cuda.hpp:129-287):
 * the rank's local tensor is cut into one box per peer rank; box p is sent to
 * (pack) or received from (unpack) peer p and lives at displs[p] elements in
 * the staging buffer, in natural order of the box's own extents -- the order
 * find_destination produces (legacy/src/tensor/shuffle_mpi_cuda.cu:42-98).
 */
typedef struct h2x_shuffle_geometry
{
    int32_t num_dims;
    int32_t elem_size;                     /* bytes per element: 2, 4 or 8 */
    int64_t local_shape[H2X_MAX_DIMS];     /* local (halo-free) extents */
    int64_t strides[H2X_MAX_DIMS];         /* element strides of the real tensor (get_strides()) */
    int64_t peer_locale_shape[H2X_MAX_DIMS]; /* process grid of the other side */
    /* rank_limits[d][j]: end, in local coordinates of dimension d, of the slab
     * that belongs to index j of the peer grid along d; concatenated over d
     * (sum of peer_locale_shape entries).  Plain limits only: the reference's
     * "-1" encoding for evenly partitioned grids of >= 16 ranks is a lookup
     * optimisation with the same meaning (shuffle_mpi_cuda.hpp:175-213). */
    const int32_t* rank_limits;
    /* displs[p]: offset (elements) of peer p's chunk, p in rank order of the
     * peer grid (dimension 0 fastest); product of peer_locale_shape entries. */
    const int32_t* displs;
} h2x_shuffle_geometry;

typedef struct h2x_shuffle_plan h2x_shuffle_plan;

/**
 * Builds the device-side box table for one geometry.  Allocates a few hundred
 * bytes of device memory and copies synchronously; call once per shuffler.
 */
int h2x_shuffle_plan_create(const h2x_shuffle_geometry* geometry, h2x_shuffle_plan** plan);
int h2x_shuffle_plan_destroy(h2x_shuffle_plan* plan);

/**
 * buffer[displs[p] + o] = tensor[box_p(o)] for every peer p.  `tensor` is the
 * get_base_ptr() of the local tensor (first interior element).  Replaces
 * pack<T, packed> (legacy/src/tensor/shuffle_mpi_cuda.cu:114-248).
 */
int h2x_shuffle_pack(const h2x_shuffle_plan* plan, const void* tensor, void* buffer, h2x_stream_t stream);

/**
 * tensor[box_p(o)] = buffer[displs[p] + o].  Replaces unpack<T, packed>
 * (legacy/src/tensor/shuffle_mpi_cuda.cu:251-372).
 */
int h2x_shuffle_unpack(const h2x_shuffle_plan* plan, void* tensor, const void* buffer, h2x_stream_t stream);

/**
 * Several ranks' pack (or unpack) steps in one launch: plan i is applied to
 * tensors[i] and buffers[i].  Pointer arrays are host memory.  For virtual
 * ranks living on one GPU; what each plan does is unchanged.
 */
int h2x_shuffle_pack_batched(const h2x_shuffle_plan* const* plans, const void* const* tensors,
                             void* const* buffers, int num_plans, h2x_stream_t stream);
int h2x_shuffle_unpack_batched(const h2x_shuffle_plan* const* plans, void* const* tensors,
                               const void* const* buffers, int num_plans, h2x_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* H2X_H_INCLUDED */
