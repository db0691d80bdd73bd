#include "host_tensor.hpp"

#include <cstring>

#include "br_hip.h"
#include "hip_tensor.hpp"

namespace br {

template <typename T>
static void print_ends(const T* d, size_t items, size_t last_dim) {
    const size_t n = std::min(last_dim, (size_t)8);
    std::cout << "--------------------------" << std::endl;
    std::cout << "First " << n << " : ";
    for (size_t i = 0; i < n; i++) std::cout << d[i] << " ";
    std::cout << std::endl;
    std::cout << "Last " << n << " : ";
    for (size_t i = 0; i < n; i++) std::cout << d[items - n + i] << " ";
    std::cout << std::endl;
}

template <DataType DT>
ComputingReturn HostTensor<DT>::io_dump(tensor_t self) {
    if (DT == DataType::Float)
        print_ends(static_cast<const float*>(mem_), self->items(), self->shape().vec().back());
    else
        print_ends(static_cast<const int*>(mem_), self->items(), self->shape().vec().back());
    return OP_OK;
}

// Block-wise raw read, 1024 elements at a time (blackriver/cpu_tensor.cpp:117-130).
template <DataType DT>
ComputingReturn HostTensor<DT>::io_load(tensor_t self, const char* fileName) {
    constexpr size_t kBlock = 1024;
    br_assert(self->items() % kBlock == 0, "Only support block read");
    std::ifstream in(fileName, std::ios::binary);
    if (!in) return OP_INPUT_ERROR;
    const size_t esize = DataType_size(DT);
    char* dst = static_cast<char*>(mem_);
    for (size_t i = 0; i < self->items() / kBlock; i++) in.read(dst + i * kBlock * esize, kBlock * esize);
    return OP_OK;
}

// Raw little-endian dump in the format io_load reads (the reference leaves
// this one unimplemented, cpu_tensor.cpp:110-114).
template <DataType DT>
ComputingReturn HostTensor<DT>::io_save(tensor_t self, const char* fileName) {
    std::ofstream out(fileName, std::ios::binary | std::ios::trunc);
    if (!out) return OP_OUTPUT_ERROR;
    out.write(static_cast<const char*>(mem_), self->items() * DataType_size(DT));
    return out.good() ? OP_OK : OP_OUTPUT_ERROR;
}

// One process is the whole world: a broadcast from ourselves leaves the data
// where it is.
template <DataType DT>
ComputingReturn HostTensor<DT>::io_mpi_bcast(tensor_t self, int root) {
    if (root != CollectiveContext::mpi_rank) return OP_INPUT_ERROR;
    return OP_OK;
}

template <DataType DT>
ComputingReturn HostTensor<DT>::io_mpi_recv(tensor_t self, int source) {
    const bool ok = CollectiveContext::take(source, CollectiveContext::mpi_rank, mem_,
                                            self->items() * DataType_size(DT));
    return ok ? OP_OK : OP_INPUT_ERROR;
}

template <DataType DT>
ComputingReturn HostTensor<DT>::io_mpi_send(tensor_t self, int dst) {
    CollectiveContext::post(CollectiveContext::mpi_rank, dst, mem_, self->items() * DataType_size(DT));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HostTensor<DT>::op_zero(tensor_t self) {
    memset(mem_, 0, self->items() * DataType_size(DT));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HostTensor<DT>::op_fill(tensor_t self, float value) {
    if (DT != DataType::Float) return OP_TODO_ERROR;
    float* d = static_cast<float*>(mem_);
    std::fill(d, d + self->items(), value);
    return OP_OK;
}

template <DataType DT>
ComputingReturn HostTensor<DT>::op_copy(tensor_t self, tensor_t src) {
    if (src->dtype() != DT) return OP_INPUT_ERROR;
    const size_t bytes = self->items() * DataType_size(DT);
    if (src->is_cpu()) {
        memmove(mem_, src->data(), bytes);
        return OP_OK;
    }
    // device -> host: the copy is complete when this returns
    BR_HIP_CHECK(br_hip_memcpy_d2h(mem_, src->data(), bytes, ComputingContext::stream));
    ComputingContext::sync();
    return OP_OK;
}

template <DataType DT>
TransformerComputing::view_result_t HostTensor<DT>::op_view(tensor_t self, size_t offset,
                                                            const std::vector<size_t>& newShape) {
    char* p = static_cast<char*>(mem_) + offset * DataType_size(DT);
    return std::make_shared<TensorType>(new HostTensor<DT>(static_cast<void*>(p)), ShapeType(newShape));
}

template struct HostTensor<DataType::Float>;
template struct HostTensor<DataType::Int>;

tensor_t create_cpu_float(std::vector<size_t>& shape_) {
    ShapeType shape(shape_);
    return std::make_shared<TensorType>(new HostTensor<DataType::Float>(shape), shape);
}

tensor_t create_cpu_int(std::vector<size_t>& shape_) {
    ShapeType shape(shape_);
    return std::make_shared<TensorType>(new HostTensor<DataType::Int>(shape), shape);
}

}  // namespace br
