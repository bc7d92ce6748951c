// Offsets for the intermediate tensors of one infer inside one device blob: tensors whose lifetimes do
// not meet share addresses.  The reference packs its "mutable blob" the same way with ov::MemorySolver
// (src/memory_manager/model/cuda_memory_model_builder.cpp:11-25, one box per tensor with the indices of
// its producing and its last consuming operation) and hands a blob to each running request from a pool
// (src/memory_manager/cuda_memory_pool.cpp:34-42); here the blob belongs to the worker thread that runs the
// request (one per stream) and grows when an infer with larger shapes needs it to.
#pragma once

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <numeric>
#include <vector>

namespace ov {
namespace hip_gpu {

struct MemoryBox {
    size_t bytes;  // > 0
    int start;     // index of the step that writes the tensor
    int end;       // index of the last step that reads it (>= start; past the last step: kept to the end of the infer)
};

// offsets[i] for boxes[i], multiples of `alignment`; returns the size of the blob.  Two boxes whose
// [start, end] ranges share a step never share an address.  Largest boxes first, each at the lowest
// address that is free for its whole lifetime: optimal for chains and layered graphs, within a small
// factor of the peak of live bytes in general.
inline size_t solve_memory(const std::vector<MemoryBox>& boxes, std::vector<size_t>& offsets, size_t alignment = 256) {
    const size_t n = boxes.size();
    offsets.assign(n, 0);
    std::vector<size_t> order(n);
    std::iota(order.begin(), order.end(), size_t(0));
    std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) {
        if (boxes[a].bytes != boxes[b].bytes) return boxes[a].bytes > boxes[b].bytes;
        return boxes[a].start < boxes[b].start;
    });
    auto aligned = [&](size_t x) { return (x + alignment - 1) / alignment * alignment; };
    std::vector<size_t> placed;
    std::vector<std::pair<size_t, size_t>> busy;  // [offset, end offset) of placed boxes alive at the same time
    size_t total = 0;
    for (size_t i : order) {
        busy.clear();
        for (size_t j : placed)
            if (boxes[j].start <= boxes[i].end && boxes[i].start <= boxes[j].end) busy.emplace_back(offsets[j], offsets[j] + aligned(boxes[j].bytes));
        std::sort(busy.begin(), busy.end());
        size_t at = 0;
        const size_t need = aligned(boxes[i].bytes);
        for (const auto& b : busy) {
            if (at + need <= b.first) break;
            at = std::max(at, b.second);
        }
        offsets[i] = at;
        total = std::max(total, at + need);
        placed.push_back(i);
    }
    return total;
}

}  // namespace hip_gpu
}  // namespace ov
