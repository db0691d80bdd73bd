// Process-wide runtime state of the host side: the compute context (device,
// one stream, scratch memory), the host bump arena that backs CPU tensors and
// a single-process stand-in for the reference's MPI/NCCL context.
//
// Same roles and boot/shutdown protocol as blackriver/context.hpp:8-47, minus
// every vendor-library handle: kernels are reached through the br_hip C ABI
// and need nothing but a stream and caller-provided workspace.
#pragma once

#include <cstddef>
#include <cstdint>
#include <deque>
#include <map>
#include <utility>
#include <vector>

namespace br {

struct ComputingContext {
    static int device;            // -1 until boot()
    static void* stream;          // the one stream every operator launches on
    static void* workspace;       // device scratch, workspace_size bytes
    static void* host_workspace;  // host scratch of the same size
    static size_t workspace_size;
    // MFMA type used when every operand of a product is stored as fp32:
    // BR_GEMM_F32 (default, fp32-faithful), BR_GEMM_F16 or BR_GEMM_BF16.
    static int fp32_gemm_compute;
    // what the most recent op_loss_backward returned (the word leaves nothing
    // on the stack; drivers read the value here)
    static float last_loss;
    // op_loss_backward prints "#################  <count> <loss>" like the
    // reference (cuda_tensor.cpp:692) unless a driver turns it off
    static bool echo_loss;
    // Gradient lift S (a power of two, 1 = off): op_loss_backward hands out
    // x_g = S * dL/dx, every backward operator passes the factor on through its
    // activation gradient and takes it out of the parameter gradients it writes
    // (1/S in the weight-gradient product's alpha and in the bias / LayerNorm
    // sums), so parameter gradients always come out at their true scale.  With
    // 16-bit products this keeps the small gradients of a mean-over-tokens loss
    // clear of fp16's subnormal range.  grad_lift_auto: op_loss_backward picks
    // S = 16 * 2^ceil(log2(count)) itself when the products run in 16 bit.
    static float grad_lift;
    static bool grad_lift_auto;
    // op_loss_backward overwrites a device-resident lm_head_g instead of adding
    // to it (set for the duration of the word op.loss_backward_set)
    static bool loss_head_overwrite;

    static void boot(int dev);  // 128 MiB of scratch like context.cpp:31
    static void shutdown();
    static bool booted() { return device >= 0; }
    static void sync();
    // Grow-only device scratch for operators whose need exceeds `workspace`
    // (the attention backward stages dP for all heads at once).
    static void* scratch(size_t bytes);
    // Grow-only device blocks of their own for 16-bit copies of fp32 GEMM
    // operands (never the workspace: operands may live there).  Slot 0 is what
    // the staged GEMM entry point converts into, slot 1 holds an operand that
    // several products of one operator share.
    static void* gemm_staging(int slot, size_t bytes);

private:
    static void* scratch_ptr_;
    static size_t scratch_size_;
    static void* staging_ptr_[2];
    static size_t staging_size_[2];
};

// One process, one GPU: rank 0 of a world of 1.  `now()` keeps feeding the
// `echo` word's "<rank>:<seconds since boot>" prefix (dag.cpp:528-533).
struct CollectiveContext {
    static int current;
    static int mpi_world;
    static int mpi_rank;
    static int nccl_rank;
    static int nccl_world;

    static void boot(int argc, char* argv[], int gpus);
    static void shutdown();
    static int now();

    // In-process mailboxes standing in for point-to-point transport so that
    // scripts that send / receive still link and run in one process.  Keyed
    // by (from, to); payloads are host copies.
    using Message = std::vector<unsigned char>;
    static void post(int from, int to, const void* data, size_t bytes);
    static bool take(int from, int to, void* data, size_t bytes);
    static void clear_mailboxes();

private:
    static std::map<std::pair<int, int>, std::deque<Message>> boxes_;
};

// Host bump allocator: one malloc at boot, page-granular blocks, never freed
// individually (context.cpp:96-121).  CPU tensors therefore need a byte size
// that is a multiple of 4096.
struct MemoryContext {
    static const size_t page_size;
    static void* root;
    static size_t total_size;
    static size_t currentp;

    static void boot(size_t total_bytes);
    static void shutdown();
    static void* alloc(size_t blk_size);
};

}  // namespace br
