/*
 * C ABI of liboeq_amd.so: runtime compilation (hiprtc) and launch of the
 * per-problem HIP kernels behind TensorProduct / TensorProductConv.
 *
 * Plain pointers and sizes only; no torch, pybind11 or C++ types cross this
 * boundary. Every function returns 0 on success or a negative oeq_status and
 * leaves a message retrievable with oeq_last_error() (thread-local). Nothing
 * in this library calls exit() or throws across the boundary.
 *
 * All device pointers must belong to the device that is current on the calling
 * thread; `stream` is a hipStream_t (NULL = the default stream). Calls only
 * enqueue work; the caller keeps the buffers alive until the stream has
 * consumed them.
 *
 * Each entry point names the reference interface it stands in for
 * (paths relative to openequivariance/openequivariance/ in the reference tree).
 */
#ifndef OEQ_AMD_H
#define OEQ_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    OEQ_OK = 0,
    OEQ_ERR_INVALID = -1,   /* bad argument (null pointer, size, role not present) */
    OEQ_ERR_COMPILE = -2,   /* hiprtc rejected the source; log in oeq_last_error() */
    OEQ_ERR_HIP = -3,       /* a HIP runtime call failed */
    OEQ_ERR_NOMEM = -4
} oeq_status;

/* ---- device properties ------------------------------------------------- */
/* Replaces DeviceProp (extension/backend/backend_hip.hpp:103-121). */
typedef struct {
    char name[256];
    char arch[64];              /* e.g. "gfx950" (feature suffixes stripped) */
    int32_t wave_size;
    int32_t compute_units;
    int32_t lds_per_block;      /* bytes */
    int32_t max_threads_per_block;
    int32_t clock_khz;
    int32_t l2_bytes;
    int64_t total_mem;          /* bytes */
} oeq_device_props;

int oeq_get_device_props(int device, oeq_device_props* out);

/* ---- runtime compilation ---------------------------------------------- */
/* Replaces HIPJITKernel::compile (extension/backend/backend_hip.hpp:217-288).
 * `arch` is explicit ("gfx950"), so this works on a host with no GPU.
 * On success *code / *code_size receive a malloc'd code object; release it
 * with oeq_free(). On OEQ_ERR_COMPILE the compiler log is the error string. */
int oeq_jit_compile(const char* source, const char* arch,
                    const char* const* options, int n_options,
                    void** code, size_t* code_size);
void oeq_free(void* p);

/* ---- a loaded set of kernels for one problem --------------------------- */
/* Replaces JITTPImpl / JITConvImpl (extension/tensorproducts.hpp:10-113,
 * extension/convolution.hpp:15-179) together with KernelProp
 * (extension/torch_core.hpp:144-178). */
typedef struct oeq_kernels oeq_kernels;

typedef enum {
    OEQ_ROLE_TP_FORWARD = 0,
    OEQ_ROLE_TP_BACKWARD = 1,
    OEQ_ROLE_CONV_FORWARD = 2,      /* main forward kernel (either mode) */
    OEQ_ROLE_CONV_BACKWARD = 3,     /* main backward kernel (either mode) */
    OEQ_ROLE_CONV_FIXUP_BACKWARD = 4,/* deterministic mode: sender-ordered segmented reduction */
    OEQ_ROLE_SEGMENT_PTR = 5,       /* builds CSR pointers from a sorted index list */
    OEQ_ROLE_FILL_ZERO = 6,         /* clears a buffer (used instead of memset: capture-safe) */
    OEQ_ROLE_TP_BACKWARD_WREDUCE = 7,/* shared weights: second pass of the weight-gradient reduction */
    OEQ_ROLE_SEGMENT_SUM = 8,       /* ordered sum of rows over the segments of a sorted key list */
    OEQ_ROLE_GROUP_COUNT = 9,       /* grouping an unsorted key list: histogram, */
    OEQ_ROLE_GROUP_SCAN = 10,       /*   exclusive scan (one block), */
    OEQ_ROLE_GROUP_SCATTER = 11,    /*   scatter of the item indices into their key's segment, */
    OEQ_ROLE_GROUP_ORDER = 12,      /*   and ascending order of the indices within each segment */
    OEQ_ROLE_DOUBLE_BACKWARD_A = 13,/* second order: gradient w.r.t. the output gradient (forward-shaped) */
    OEQ_ROLE_DOUBLE_BACKWARD_B = 14,/* second order: gradients w.r.t. X, Y, W (backward-shaped) */
    OEQ_ROLE_ORDER_HOP = 15,        /* convolution walk order: one hop of the node clustering */
    OEQ_ROLE_HUB_COUNT = 16,        /* long edge segments cut into chunks: extra walk positions per node, */
    OEQ_ROLE_HUB_FILL = 17,         /*   and the list of those positions */
    OEQ_ROLE_CONV_FIXUP_FORWARD = 18,/* adds the rows written by the extra chunks to their nodes' rows, in chunk order */
    OEQ_ROLE_CONV_BACKWARD_DX = 19, /* OEQ_DX_SENDER_WALK: the sender gradients by a walk over the senders' edge segments
                                       (forward-shaped: argument list of OEQ_ROLE_CONV_FORWARD with dZ for X, the
                                       receivers for the senders and the sender-side index) */
    OEQ_ROLE_COUNT = 20
} oeq_role;

/* How the convolution kernels of a set find the edges of a node (oeq_problem_dims.deterministic):
 * the reference has the first two (loop_unroll_conv_atomic.cuh / loop_unroll_conv_det.cuh). */
typedef enum {
    OEQ_CONV_ATOMIC = 0,   /* any edge order; contiguous edge ranges per wave, float atomics at every change of node */
    OEQ_CONV_SORTED = 1,   /* caller passes receiver-sorted edges (+ sender-major permutation for backward); CSR walk,
                              fixed summation order, no atomics on node data */
    OEQ_CONV_GROUPED = 2   /* any edge order; the library groups the edge indices by receiver (and by sender for
                              backward) on the device, ascending within a group, then runs the same CSR walk
                              through that index: fixed summation order for a given edge list, no atomics on node
                              data */
} oeq_conv_mode;

/* What the receiver walk of the convolution backward does with the per-edge terms of the gradient
 * with respect to the sender rows (oeq_problem_dims.dx_mode). The reference's deterministic backward
 * walks sender-sorted edges instead and re-reads the receiver's gradient row per edge
 * (loop_unroll_conv_det.cuh:187-293). */
typedef enum {
    OEQ_DX_TERMS = 0,    /* terms go to scratch; fixup_backward sums them per sender in sender-major order */
    OEQ_DX_ATOMIC = 1,   /* terms are added into the cleared sender rows with float atomics (not bit-reproducible) */
    OEQ_DX_ARRIVAL = 2,  /* terms go to scratch; the wave that delivers the last term of a sender sums that
                            sender's terms in sender-major order (same bits as OEQ_DX_TERMS, no second kernel) */
    OEQ_DX_SENDER_WALK = 3 /* no terms: OEQ_ROLE_CONV_BACKWARD_DX walks every sender's edges in sender-major order
                            and forms its gradient row from dZ of the receivers, Y and W (this is the reference's
                            scheme, loop_unroll_conv_det.cuh:187-293; chosen where rows of X are long and rows of dZ
                            short) */
} oeq_dx_mode;

/* Several descriptors may name the same role: those kernels are launched back to back, in
 * descriptor order, with the same arguments and launch shape (that of the last descriptor). */
typedef struct {
    int32_t role;               /* oeq_role */
    const char* kernel_name;    /* __global__ symbol (extern "C") in the code object */
    uint32_t block_threads;
    uint32_t units_per_block;   /* rows / nodes / edges one block handles per sweep */
    uint32_t max_blocks;        /* 0 = one block per ceil(units/units_per_block) */
    uint32_t grid_multiple;     /* 0/1 = none; else the grid is rounded up to a multiple of this (kernels that
                                   remap blockIdx so that each XCD walks a contiguous range of units) */
} oeq_kernel_desc;

typedef struct {
    int64_t L1_dim, L2_dim, L3_dim, weight_numel;
    int32_t elem_size;          /* 4 = float, 8 = double (irreps and weights alike) */
    int32_t shared_weights;     /* weights are [weight_numel] instead of [rows, weight_numel] */
    int32_t deterministic;      /* conv: an oeq_conv_mode value */
    int32_t wpartial_per_block; /* shared weights: partial weight-gradient rows each block of the
                                   backward kernel writes (0 = none); the workspace holds
                                   max_blocks * wpartial_per_block rows of weight_numel elements */
    int32_t dx_mode;            /* conv backward, walk modes: an oeq_dx_mode value */
    int32_t n_chunks;           /* conv backward, OEQ_DX_ARRIVAL: arrival counters per sender node
                                   (one per 64-channel chunk of a row) */
    int32_t order_hops;         /* conv, walk modes: > 0 = at every call the nodes are clustered by the
                                   highest-priority node within this many edges and walked cluster by cluster,
                                   so that nodes sharing senders run side by side and the gathered sender rows
                                   are served by the L2; 0 = nodes are walked by index */
    int32_t hub_limit;          /* conv, walk modes: > 0 = a node with more edges than this is walked in chunks of
                                   this many edges by different wave groups (the first chunk at the node's own walk
                                   position, the others at extra positions listed in the index), so that the time
                                   of a call does not grow with the largest degree: forward-shaped kernels write
                                   the extra chunks to scratch rows that fixup_forward adds to the node's row in
                                   chunk order; 0 = every segment is walked whole. Plays the role of the
                                   reference's equal edge ranges per warp with fixup_forward
                                   (templates/loop_unroll_conv_det.cuh:34-66, 96-179,
                                   core/LoopUnrollConv.py:142-185). */
} oeq_problem_dims;

/* `code` is a code object as oeq_jit_compile returns it, or a pack of several (the kernels of a large set
 * compiled side by side, in different processes; every kernel in exactly one of them): the 8 bytes "OEQPACK1",
 * a uint64 count, that many uint64 byte sizes, then the code objects in that order, each starting at the next
 * multiple of 64 bytes from the start of the pack (little endian). Kernel names are looked up in all of them.
 * No counterpart in the reference, whose kernel sets are one NVRTC / hiprtc program each
 * (extension/backend/backend_hip.hpp:217-288). */
int oeq_kernels_create(const void* code, size_t code_size,
                       const oeq_problem_dims* dims,
                       const oeq_kernel_desc* descs, int n_descs,
                       oeq_kernels** out);
void oeq_kernels_destroy(oeq_kernels* k);

/* ---- batched tensor product ------------------------------------------- */
/* Replaces JITTPImpl::exec_tensor_product (extension/tensorproducts.hpp:75-85)
 * as called by jit_tp_forward (extension/torch_core.hpp:274-310).
 * L1_in [num_batch, L1_dim], L2_in [num_batch, L2_dim],
 * W [num_batch, weight_numel] or [weight_numel], L3_out [num_batch, L3_dim]
 * (every element is overwritten). */
int oeq_tp_forward(oeq_kernels* k, int64_t num_batch,
                   const void* L1_in, const void* L2_in, const void* W,
                   void* L3_out, void* stream);

/* Replaces JITTPImpl::backward (extension/tensorproducts.hpp:87-95) as called
 * by jit_tp_backward (extension/torch_core.hpp:312-355). All three gradients
 * are fully overwritten. With shared weights `workspace` must hold
 * oeq_tp_backward_workspace_bytes() bytes (partial weight gradients, reduced
 * in a fixed order: no atomics); otherwise it may be NULL. */
int oeq_tp_backward(oeq_kernels* k, int64_t num_batch,
                    const void* L1_in, void* L1_grad,
                    const void* L2_in, void* L2_grad,
                    const void* W, void* W_grad,
                    const void* L3_grad,
                    void* workspace, size_t workspace_bytes, void* stream);
size_t oeq_tp_backward_workspace_bytes(const oeq_kernels* k, int64_t num_batch);

/* ---- fused graph convolution ------------------------------------------ */
/* Replaces JITConvImpl::exec_conv (extension/convolution.hpp:78-107) as called
 * by jit_conv_forward (extension/torch_core.hpp:422-476).
 * L1_in [node_count, L1_dim], L2_in [nnz, L2_dim], W [nnz, weight_numel] or
 * [weight_numel], rows/cols int64 [nnz] (rows = receiver, cols = sender),
 * L3_out [node_count, L3_dim] (cleared and fully written by this call).
 * Deterministic mode requires rows sorted ascending and a workspace of
 * oeq_conv_forward_workspace_bytes() bytes. */
int oeq_conv_forward(oeq_kernels* k, int64_t node_count, int64_t nnz,
                     const void* L1_in, const void* L2_in, const void* W,
                     void* L3_out, const int64_t* rows, const int64_t* cols,
                     void* workspace, size_t workspace_bytes, void* stream);
/* index + scratch (the rows of extra chunks, see oeq_problem_dims.hub_limit; sized for nnz / hub_limit of them) */
size_t oeq_conv_forward_workspace_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz);

/* oeq_conv_forward for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc. It has no counterpart in the reference (whose convolution always takes a
 * caller-allocated workspace tensor). Same operands and result as oeq_conv_forward; the index scratch
 * (CSR pointers, edge grouping, walk order) lives in a device array inside the library instead of a
 * caller workspace, and the call itself allocates nothing (no hipMalloc / hipFree, no event or module
 * creation): the kernel set must already be loaded on the current device, i.e. oeq_conv_forward has run on
 * it once. Limits: the scratch needed, oeq_conv_forward_workspace_bytes(), must not exceed
 * oeq_static_scratch_bytes() (32 MiB: e.g. 1.85 M edges over 50 000 nodes with deterministic=False, 590 000
 * nodes in deterministic mode, where the index and the temporaries of its build take 56 bytes per node);
 * larger calls are refused with OEQ_ERR_INVALID. Every call on a GPU uses
 * that GPU's one array: calls that overlap in time on one GPU (two streams, two threads) race and must be
 * serialised by the caller. Long edge segments are walked whole here (oeq_problem_dims.hub_limit is not
 * applied: the rows of extra chunks would need scratch of their own), so the sum over a hub node's edges is
 * formed in one pass and can differ in the last bits from oeq_conv_forward's. Per-kernel timing (oeq_kernel_timing_enable) is not applied to these calls. */
int oeq_conv_forward_static(oeq_kernels* k, int64_t node_count, int64_t nnz,
                            const void* L1_in, const void* L2_in, const void* W,
                            void* L3_out, const int64_t* rows, const int64_t* cols,
                            void* stream);
size_t oeq_static_scratch_bytes(void);

/* Replaces JITConvImpl::backward (extension/convolution.hpp:109-136) as called
 * by jit_conv_backward (extension/torch_core.hpp:478-542). Deterministic mode
 * additionally needs transpose_perm [nnz]: the permutation listing the
 * (row-sorted) edges in sender-major order; it is ignored in atomic mode. */
int oeq_conv_backward(oeq_kernels* k, int64_t node_count, int64_t nnz,
                      const void* L1_in, void* L1_grad,
                      const void* L2_in, void* L2_grad,
                      const void* W, void* W_grad,
                      const void* L3_grad,
                      const int64_t* rows, const int64_t* cols,
                      const int64_t* transpose_perm,
                      void* workspace, size_t workspace_bytes, void* stream);
size_t oeq_conv_backward_workspace_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz);

/* ---- the index of an edge list, built once and used by several calls --------------------------------- */
/* Every walk-mode convolution call first derives an index from (rows, cols): CSR pointers over receivers,
 * in OEQ_CONV_GROUPED mode the edge ids grouped by receiver, the walk order of the nodes and, with
 * `sender_side` != 0, the same over senders (needed by the calls that reduce per-edge sender-gradient terms:
 * oeq_conv_backward unless oeq_problem_dims.dx_mode is OEQ_DX_ATOMIC, and oeq_conv_double_backward). The entry
 * points above build it into the front of their workspace at every call. A caller that runs several
 * convolutions over one edge list (forward and backward of every layer of a model) builds it once with
 * oeq_conv_index_build and passes it to the *_indexed variants, which take the same operands, `index` /
 * `index_bytes` / `index_sender_side` as given to the build, and a scratch buffer of
 * oeq_conv_forward_scratch_bytes() / oeq_conv_backward_scratch_bytes() / oeq_conv_double_backward_scratch_bytes().
 * The reference keeps the corresponding state (its workspace tensor and, for the deterministic mode, the
 * caller's transpose_perm) in the Python module (_torch/TensorProductConv.py:187-193). The index is read-only
 * after the build, so calls on several streams may share it once the build has completed; it is tied to the
 * kernel set's mode, node_count, nnz and the contents of rows / cols (/ transpose_perm). For OEQ_CONV_ATOMIC
 * kernel sets there is no index (size 0; pass NULL). */
size_t oeq_conv_index_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz, int sender_side);
int oeq_conv_index_build(oeq_kernels* k, int64_t node_count, int64_t nnz,
                         const int64_t* rows, const int64_t* cols, const int64_t* transpose_perm,
                         int sender_side, void* index, size_t index_bytes, void* stream);
/* Where a piece of a built index lies, for inspection (tests, tools): byte offset into the index buffer and
 * number of int64 entries. No counterpart in the reference. */
typedef enum {
    OEQ_INDEX_ROWPTR = 0,    /* CSR pointers over receivers, node_count + 1 */
    OEQ_INDEX_COLPTR = 1,    /* ... over senders (sender side) */
    OEQ_INDEX_RPERM = 2,     /* OEQ_CONV_GROUPED: edge ids grouped by receiver, nnz */
    OEQ_INDEX_SPERM = 3,     /* ... by sender (sender side) */
    OEQ_INDEX_ORDER = 4,     /* walk order of the nodes, node_count */
    OEQ_INDEX_HUBPTR = 5,    /* first extra walk position of every node, node_count + 1 (hub_limit > 0) */
    OEQ_INDEX_HUBNODE = 6,   /* node of every extra walk position, nnz / hub_limit */
    OEQ_INDEX_SHUBPTR = 7,   /* the same two over the senders' segments (sender side) */
    OEQ_INDEX_SHUBNODE = 8
} oeq_index_piece;
int oeq_conv_index_piece(const oeq_kernels* k, int64_t node_count, int64_t nnz, int sender_side, int piece,
                         size_t* offset, size_t* entries);
int oeq_conv_forward_indexed(oeq_kernels* k, int64_t node_count, int64_t nnz,
                             const void* L1_in, const void* L2_in, const void* W, void* L3_out,
                             const int64_t* rows, const int64_t* cols,
                             const void* index, size_t index_bytes, int index_sender_side,
                             void* scratch, size_t scratch_bytes, void* stream);
size_t oeq_conv_forward_scratch_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz);
int oeq_conv_backward_indexed(oeq_kernels* k, int64_t node_count, int64_t nnz,
                              const void* L1_in, void* L1_grad, const void* L2_in, void* L2_grad,
                              const void* W, void* W_grad, const void* L3_grad,
                              const int64_t* rows, const int64_t* cols, const int64_t* transpose_perm,
                              const void* index, size_t index_bytes, int index_sender_side,
                              void* scratch, size_t scratch_bytes, void* stream);
size_t oeq_conv_backward_scratch_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz);
int oeq_conv_double_backward_indexed(oeq_kernels* k, int64_t node_count, int64_t nnz,
                                     const void* L1_in, const void* L2_in, const void* W, const void* L3_grad,
                                     const void* L1_dgrad, const void* L2_dgrad, const void* W_dgrad,
                                     void* L1_grad, void* L2_grad, void* W_grad, void* L3_dgrad,
                                     const int64_t* rows, const int64_t* cols, const int64_t* transpose_perm,
                                     const void* index, size_t index_bytes,
                                     void* scratch, size_t scratch_bytes, void* stream);
size_t oeq_conv_double_backward_scratch_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz);

/* ---- second-order ('double backward') kernels ---------------------------- */
/* Gradient of the backward pass: given the operands of oeq_tp_backward (L1_in, L2_in, W, L3_grad) and
 * cotangents L1_dgrad, L2_dgrad, W_dgrad of its three results, writes the gradients with respect to
 * L1_in, L2_in, W and L3_grad (all four fully overwritten). Replaces JITTPImpl::double_backward
 * (extension/tensorproducts.hpp:97-111) as called by jit_tp_double_backward
 * (extension/torch_core.hpp:357-420). Only kernel sets for which oeq_has_double_backward() is non-zero
 * carry these kernels (by default every batch kernel set, and the convolutions with per-edge weights); for the
 * others the same result is composed from oeq_tp_forward / oeq_tp_backward calls by the caller. */
int oeq_has_double_backward(const oeq_kernels* k);
int oeq_tp_double_backward(oeq_kernels* k, int64_t num_batch,
                           const void* L1_in, const void* L2_in, const void* W, const void* L3_grad,
                           const void* L1_dgrad, const void* L2_dgrad, const void* W_dgrad,
                           void* L1_grad, void* L2_grad, void* W_grad, void* L3_dgrad,
                           void* workspace, size_t workspace_bytes, void* stream);
/* Workspace of oeq_tp_double_backward: partial weight gradients for shared weights (summed in a fixed
 * order by a second kernel, as in oeq_tp_backward); zero for per-row weights, and then workspace may be NULL. */
size_t oeq_tp_double_backward_workspace_bytes(const oeq_kernels* k, int64_t num_batch);

/* The same for the fused convolution; replaces JITConvImpl::double_backward
 * (extension/convolution.hpp:138-178) as called by jit_conv_double_backward
 * (extension/torch_core.hpp:544-625). Index arguments are those of oeq_conv_backward; the workspace must
 * hold oeq_conv_double_backward_workspace_bytes() bytes. Not available for OEQ_CONV_ATOMIC kernel sets. */
int oeq_conv_double_backward(oeq_kernels* k, int64_t node_count, int64_t nnz,
                             const void* L1_in, const void* L2_in, const void* W, const void* L3_grad,
                             const void* L1_dgrad, const void* L2_dgrad, const void* W_dgrad,
                             void* L1_grad, void* L2_grad, void* W_grad, void* L3_dgrad,
                             const int64_t* rows, const int64_t* cols, const int64_t* transpose_perm,
                             void* workspace, size_t workspace_bytes, void* stream);
size_t oeq_conv_double_backward_workspace_bytes(const oeq_kernels* k, int64_t node_count, int64_t nnz);

/* ---- ordered segment sum -------------------------------------------------- */
/* dst[s, :] = sum, in list order, of src[item, :] over the items whose key is s, for s < n_segments.
 * The list is 0..n_items-1, or perm[0..n_items-1] when perm != NULL, and keys must be non-decreasing
 * along it. Rows have row_len elements of the kernel set's element type. Deterministic (no atomics).
 * Replaces the reference's scatter_add_wrapper (core/ConvolutionBase.py:292-301) where a fixed
 * summation order is wanted; used by the unfused 'uvw' convolution. The workspace must hold
 * oeq_segment_sum_workspace_bytes() bytes. */
int oeq_segment_sum(oeq_kernels* k, int64_t n_segments, int64_t n_items, int64_t row_len,
                    const void* src, void* dst, const int64_t* keys, const int64_t* perm,
                    void* workspace, size_t workspace_bytes, void* stream);
size_t oeq_segment_sum_workspace_bytes(const oeq_kernels* k, int64_t n_segments);

/* Same sum for keys in ANY order: the item indices are first grouped by key on the device (ascending
 * within a key, so the summation order depends on the key list only), then summed as above. Replaces the
 * same scatter_add_wrapper call where the reference relies on float atomics. */
int oeq_grouped_sum(oeq_kernels* k, int64_t n_segments, int64_t n_items, int64_t row_len,
                    const void* src, void* dst, const int64_t* keys,
                    void* workspace, size_t workspace_bytes, void* stream);
size_t oeq_grouped_sum_workspace_bytes(const oeq_kernels* k, int64_t n_segments, int64_t n_items);

/* ---- per-kernel timing --------------------------------------------------- */
/* Replaces GPUTimer (extension/backend/backend_hip.hpp:67-101). While enabled,
 * every kernel this set launches is bracketed by HIP events on the stream it is
 * launched on. oeq_kernel_timing_collect() waits for the recorded launches of
 * `role`, returns their summed duration and count, and forgets them. */
int oeq_kernel_timing_enable(oeq_kernels* k, int enable);
int oeq_kernel_timing_collect(oeq_kernels* k, int role, double* total_ms, int64_t* launches);

/* ---- diagnostics -------------------------------------------------------- */
const char* oeq_last_error(void);
int oeq_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* OEQ_AMD_H */
