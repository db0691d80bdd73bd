// HostTensor: CPU-resident storage for fp32 and int32 tensors.
//
// Storage and transport only, exactly the role CPUTensor has in the reference
// (blackriver/cpu_tensor.hpp:30-39): creation in the host arena, zero / fill /
// copy / view, file load, dump and the control-plane transport.  There are no
// math operators on the CPU: calling one falls through to OP_TODO_ERROR and
// panics, on purpose.
#pragma once

#include "computing.hpp"
#include "runtime.hpp"
#include "tensor.hpp"

namespace br {

template <DataType DT>
struct HostTensor : public TransformerComputing {
    static_assert(DT == DataType::Float || DT == DataType::Int, "host tensors are fp32 or int32");

    // owning constructor: a page-granular block from MemoryContext
    explicit HostTensor(const ShapeType& shape) : mem_(MemoryContext::alloc(shape.numel() * DataType_size(DT))) {}
    // borrowing constructor (views)
    explicit HostTensor(void* mem) : mem_(mem) {}
    ~HostTensor() override = default;

    void* data() { return mem_; }

    ComputingReturn io_dump(tensor_t self) override;
    ComputingReturn io_load(tensor_t self, const char* fileName) override;
    ComputingReturn io_save(tensor_t self, const char* fileName) override;
    ComputingReturn io_mpi_bcast(tensor_t self, int root) override;
    ComputingReturn io_mpi_recv(tensor_t self, int source) override;
    ComputingReturn io_mpi_send(tensor_t self, int dst) override;

    ComputingReturn op_zero(tensor_t self) override;
    ComputingReturn op_fill(tensor_t self, float value) override;
    ComputingReturn op_copy(tensor_t self, tensor_t src) override;
    view_result_t op_view(tensor_t self, size_t offset, const std::vector<size_t>& newShape) override;

private:
    void* mem_;
};

}  // namespace br
