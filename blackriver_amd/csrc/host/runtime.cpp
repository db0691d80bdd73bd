#include "runtime.hpp"

#include <cstdlib>
#include <cstring>
#include <ctime>

#include "br_hip.h"
#include "common.hpp"

namespace br {

// ---------------------------------------------------------------- panics
static PanicHook g_hook = nullptr;

void set_panic_hook(PanicHook hook) { g_hook = hook; }

void panic_at(const char* file, int line, const std::string& msg) {
    std::string text = "**Panic:\t" + msg + "\nSource:\t\t" + file + ", line " + std::to_string(line) + "\n";
    if (g_hook) {
        g_hook(text);
    }
    std::cerr << text;
    abort();
}

void assert_at(const char* expr, bool ok, const char* file, int line, const char* msg) {
    if (ok) return;
    std::string text = std::string("**Assert failed:\t") + msg + "\nExpected:\t" + expr + "\nSource:\t\t" + file +
                       ", line " + std::to_string(line) + "\n";
    if (g_hook) {
        g_hook(text);
    }
    std::cerr << text;
    abort();
}

void hip_check_at(const char* what, int code, const char* file, int line) {
    if (code == 0) return;
    std::string text = std::string("[") + file + ":" + std::to_string(line) + "] `" + what +
                       "` returns error: " + std::to_string(code) + " (" + br_hip_error_string(code) + ").\n";
    if (g_hook) {
        g_hook(text);
    }
    std::cerr << text;
    exit(1);
}

// ------------------------------------------------------ ComputingContext
int ComputingContext::device = -1;
void* ComputingContext::stream = nullptr;
void* ComputingContext::workspace = nullptr;
void* ComputingContext::host_workspace = nullptr;
size_t ComputingContext::workspace_size = 0;
int ComputingContext::fp32_gemm_compute = BR_GEMM_F32;
float ComputingContext::last_loss = 0.0f;
bool ComputingContext::echo_loss = true;
float ComputingContext::grad_lift = 1.0f;
bool ComputingContext::grad_lift_auto = false;
bool ComputingContext::loss_head_overwrite = false;
void* ComputingContext::scratch_ptr_ = nullptr;
size_t ComputingContext::scratch_size_ = 0;
void* ComputingContext::staging_ptr_[2] = {nullptr, nullptr};
size_t ComputingContext::staging_size_[2] = {0, 0};

void ComputingContext::boot(int dev) {
    br_assert(device < 0, "ComputingContext is already booted");
    BR_HIP_CHECK(br_hip_set_device(dev));
    BR_HIP_CHECK(br_hip_stream_create(&stream));
    workspace_size = static_cast<size_t>(1024) * 1024 * 32 * 4;
    BR_HIP_CHECK(br_hip_malloc(&workspace, workspace_size));
    host_workspace = malloc(workspace_size);
    br_assert(host_workspace != nullptr, "can't allocate the host workspace");
    device = dev;
}

void ComputingContext::shutdown() {
    if (device < 0) return;
    sync();
    free(host_workspace);
    if (scratch_ptr_) BR_HIP_CHECK(br_hip_free(scratch_ptr_));
    for (int i = 0; i < 2; i++) {
        if (staging_ptr_[i]) BR_HIP_CHECK(br_hip_free(staging_ptr_[i]));
        staging_ptr_[i] = nullptr;
        staging_size_[i] = 0;
    }
    BR_HIP_CHECK(br_hip_free(workspace));
    BR_HIP_CHECK(br_hip_stream_destroy(stream));
    host_workspace = workspace = stream = scratch_ptr_ = nullptr;
    workspace_size = scratch_size_ = 0;
    device = -1;
}

void ComputingContext::sync() {
    br_assert(device >= 0, "ComputingContext is not booted");
    BR_HIP_CHECK(br_hip_stream_sync(stream));
}

void* ComputingContext::scratch(size_t bytes) {
    br_assert(device >= 0, "ComputingContext is not booted");
    if (bytes <= workspace_size) return workspace;
    if (bytes > scratch_size_) {
        // earlier kernels on the stream may still be using the old block
        sync();
        if (scratch_ptr_) BR_HIP_CHECK(br_hip_free(scratch_ptr_));
        BR_HIP_CHECK(br_hip_malloc(&scratch_ptr_, bytes));
        scratch_size_ = bytes;
    }
    return scratch_ptr_;
}

void* ComputingContext::gemm_staging(int slot, size_t bytes) {
    br_assert(device >= 0, "ComputingContext is not booted");
    br_assert(slot == 0 || slot == 1, "staging slot");
    if (bytes > staging_size_[slot]) {
        // earlier kernels on the stream may still be using the old block
        sync();
        if (staging_ptr_[slot]) BR_HIP_CHECK(br_hip_free(staging_ptr_[slot]));
        // room to spare, so that a slightly larger product does not reallocate
        bytes += bytes / 4;
        BR_HIP_CHECK(br_hip_malloc(&staging_ptr_[slot], bytes));
        staging_size_[slot] = bytes;
    }
    return staging_ptr_[slot];
}

// ----------------------------------------------------- CollectiveContext
int CollectiveContext::current = -1;
int CollectiveContext::mpi_world = 1;
int CollectiveContext::mpi_rank = 0;
int CollectiveContext::nccl_rank = 0;
int CollectiveContext::nccl_world = 1;
std::map<std::pair<int, int>, std::deque<CollectiveContext::Message>> CollectiveContext::boxes_;

void CollectiveContext::boot(int, char**, int gpus) {
    current = static_cast<int>(time(nullptr));
    br_assert(gpus == 1, "this build runs every layer on one GPU in one process");
    mpi_world = 1;
    mpi_rank = 0;
    nccl_world = 1;
    nccl_rank = 0;
}

void CollectiveContext::shutdown() { clear_mailboxes(); }

int CollectiveContext::now() {
    if (current < 0) current = static_cast<int>(time(nullptr));
    return static_cast<int>(time(nullptr)) - current;
}

void CollectiveContext::post(int from, int to, const void* data, size_t bytes) {
    Message m(bytes);
    memcpy(m.data(), data, bytes);
    boxes_[{from, to}].push_back(std::move(m));
}

bool CollectiveContext::take(int from, int to, void* data, size_t bytes) {
    auto it = boxes_.find({from, to});
    if (it == boxes_.end() || it->second.empty()) return false;
    br_assert(it->second.front().size() == bytes, "received message has a different size");
    memcpy(data, it->second.front().data(), bytes);
    it->second.pop_front();
    return true;
}

void CollectiveContext::clear_mailboxes() { boxes_.clear(); }

// --------------------------------------------------------- MemoryContext
const size_t MemoryContext::page_size = 4096;
void* MemoryContext::root = nullptr;
size_t MemoryContext::total_size = 0;
size_t MemoryContext::currentp = 0;

void MemoryContext::boot(size_t total_bytes) {
    br_assert(root == nullptr, "MemoryContext is already booted");
    root = malloc(total_bytes);
    br_assert(root != nullptr, "can't allocate the host arena");
    total_size = total_bytes;
    currentp = 0;
}

void MemoryContext::shutdown() {
    free(root);
    root = nullptr;
    total_size = currentp = 0;
}

void* MemoryContext::alloc(size_t blk_size) {
    br_assert(blk_size % page_size == 0, "block size must page aligend");
    if (blk_size + currentp > total_size) {
        std::cout << CollectiveContext::mpi_rank << ": " << currentp << " " << blk_size << std::endl;
        br_panic("Can't allocate memory, out of pre-allocating");
    }
    void* ret = static_cast<unsigned char*>(root) + currentp;
    currentp += blk_size;
    return ret;
}

}  // namespace br
