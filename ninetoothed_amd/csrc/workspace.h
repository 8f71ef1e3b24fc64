// Device scratch buffers that outlive a call.
//
// conv2d's repacked operands, the narrowed K / V of fp32 attention, the partial products of
// split-K GEMMs and the dense copies of GEMM operands that the direct-to-LDS kernels cannot read in place
// are temporaries of up to tens of megabytes.  Taking them from the stream-ordered allocator at every call leaves the
// GPU idle for ~10 us between calls (the allocation that follows a pending free is not handed
// out before the free has executed).  Instead the library keeps one buffer per (device, stream,
// purpose), grows it when a call needs more, and reuses it otherwise: work on one stream
// executes in order, so the next call may overwrite what the previous call has finished with.
// Buffers are released by nt_release_workspaces() or at process exit.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>

namespace nt {

enum WorkspacePurpose {
    kWorkspaceConvInput, kWorkspaceConvFilter, kWorkspaceAttentionNarrow, kWorkspaceGemmParts, kWorkspaceAttentionParts,
    kWorkspaceGemmLhsWidened, kWorkspaceGemmRhsWidened, kWorkspaceGemmBiasWidened, kWorkspaceGemmLhsDense, kWorkspaceGemmRhsDense,
    kWorkspaceAttentionPaddedQ, kWorkspaceAttentionPaddedK, kWorkspaceAttentionPaddedV, kWorkspaceAttentionPaddedO, kWorkspaceSoftmaxParts, kWorkspacePurposes
};

// Holds the registry lock from construction to destruction: create it, take the buffers,
// enqueue every kernel that uses them, then let it go.  Two host threads that launch on the
// same stream then cannot interleave their kernels on a shared buffer.  A thread may hold
// several leases at once (a caller that keeps its own buffers alive across a call that takes more).
class WorkspaceLease {
public:
    explicit WorkspaceLease(hipStream_t stream);
    ~WorkspaceLease();
    WorkspaceLease(const WorkspaceLease &) = delete;
    WorkspaceLease &operator=(const WorkspaceLease &) = delete;

    // A buffer of at least `bytes` (256-byte aligned), or nullptr when it cannot be allocated
    // (out of memory, or the stream is being captured into a graph and no buffer of that size
    // exists yet: growing synchronises the device).
    void *get(WorkspacePurpose purpose, size_t bytes);

private:
    hipStream_t stream_;
    int device_;
};

}  // namespace nt
