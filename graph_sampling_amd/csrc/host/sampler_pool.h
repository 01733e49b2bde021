#pragma once
#include <torch/torch.h>

#include <vector>

#include "graph.h"

namespace gs {

// GraphSAGE-style minibatches sampled side by side by `workers` host threads, one stream
// each.  Per minibatch, for every layer in turn: fused column slice + uniform sample of the
// current seeds, relabel, next seeds = frontier.  Returns per minibatch the flat list
// [frontier, offsets, indices] x layers (what Graph::Relabel returns for a CSC block).
// Minibatch i draws with seeds first_seed + i * layers + layer whatever thread runs it.
std::vector<std::vector<torch::Tensor>> SampleBlocks(const c10::intrusive_ptr<Graph>& graph,
                                                     std::vector<torch::Tensor> seed_sets,
                                                     std::vector<int64_t> fanouts, bool replace,
                                                     int64_t workers, int64_t first_seed);

// The same pool with a super-batch per task: the seed sets go `per_call` at a time through
// Graph::QueueSampleLayersBatched, a thread queues its next group before it collects the one
// before (`workers` must be 1 for now: super-batches side by side are switched off).  Group g (seed sets g * per_call ...) draws with
// the seeds first_seed + g * per_call * layers + layer whatever thread runs it.
std::vector<std::vector<torch::Tensor>> SampleBlocksBatched(
    const c10::intrusive_ptr<Graph>& graph, std::vector<torch::Tensor> seed_sets,
    std::vector<int64_t> fanouts, bool replace, int64_t workers, int64_t per_call,
    int64_t first_seed);

}  // namespace gs
