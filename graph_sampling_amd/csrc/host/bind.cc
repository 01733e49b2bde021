// TORCH_LIBRARY registration: torch.classes.gs_classes.{Graph, HeteroGraph} and
// torch.ops.gs_ops.*.  Every method is registered under the CamelCase name the
// reference's src/pybind.cc:12-86 uses and under the snake_case name its Python
// package and examples call (python/gs/matrix_api/matrix.py); both reach the
// same C++ method.
#include <torch/custom_class.h>
#include <torch/script.h>

#include "graph.h"
#include "graph_ops.h"
#include "hetero_graph.h"
#include "hip_ops.h"
#include "sampler_pool.h"
#include "tensor_ops.h"

using namespace gs;

namespace {
void SetSeed(int64_t seed) { hip::SetSeed(static_cast<uint64_t>(seed)); }
void SetThreadSeed(int64_t seed) { hip::SetThreadSeed(static_cast<uint64_t>(seed)); }
void SetSampleAlgo(int64_t algo) { hip::SetSampleAlgo(algo); }
void SetOrderedSums(bool on) { hip::SetOrderedSums(on); }
void SetBatchedNoWait(bool on) { hip::SetBatchedNoWait(on); }
std::vector<int64_t> BatchedNoWaitCounts() { return hip::BatchedNoWaitCounts(); }
void SetDeferredSampling(bool on) { hip::SetDeferredSampling(on); }
void DebugRaiseLookbackError(torch::Tensor like) { hip::DebugRaiseLookbackError(like); }
torch::Tensor UniqueOp(torch::Tensor ids) { return TensorUnique(ids); }
}  // namespace

#define GS_DEF2(camel, snake, fn) .def(camel, fn).def(snake, fn)

TORCH_LIBRARY(gs_classes, m) {
  // not in the reference: a minibatch whose launches are queued and whose results are
  // collected later (Graph::QueueSampleLayers)
  m.class_<QueuedLayers>("QueuedLayers") GS_DEF2("_CAPI_Collect", "collect", &QueuedLayers::Collect);
  // the same for a super-batch (Graph::QueueSampleLayersBatched)
  m.class_<QueuedSuperBatch>("QueuedSuperBatch")
      GS_DEF2("_CAPI_Collect", "collect", &QueuedSuperBatch::Collect);

  m.class_<Graph>("Graph")
      .def(torch::init<bool>())
      GS_DEF2("_CAPI_SetData", "_CAPI_set_data", &Graph::SetData)
      GS_DEF2("_CAPI_GetData", "_CAPI_get_data", &Graph::GetData)
      GS_DEF2("_CAPI_GetNumRows", "_CAPI_get_num_rows", &Graph::GetNumRows)
      GS_DEF2("_CAPI_GetNumCols", "_CAPI_get_num_cols", &Graph::GetNumCols)
      GS_DEF2("_CAPI_GetNumEdges", "_CAPI_get_num_edges", &Graph::GetNumEdges)
      GS_DEF2("_CAPI_Slicing", "_CAPI_slicing", &Graph::Slicing)
      GS_DEF2("_CAPI_Sampling", "_CAPI_sampling", &Graph::Sampling)
      GS_DEF2("_CAPI_SamplingWithProbs", "_CAPI_sampling_with_probs", &Graph::SamplingProbs)
      GS_DEF2("_CAPI_FusedColumnwiseSlicingSampling", "_CAPI_fused_columnwise_slicing_sampling",
              &Graph::ColumnwiseFusedSlicingAndSampling)
      // not in the reference: the per-layer loop of its GraphSAGE examples as one call
      GS_DEF2("_CAPI_SampleLayers", "_CAPI_sample_layers", &Graph::SampleLayers)
      GS_DEF2("_CAPI_SampleLayersIfQueued", "_CAPI_sample_layers_if_queued",
              &Graph::SampleLayersIfQueued)
      // not in the reference: its super-batch flow (examples/graphsage/batching.py:59-98) as one call
      GS_DEF2("_CAPI_SampleLayersBatched", "_CAPI_sample_layers_batched",
              &Graph::SampleLayersBatched)
      GS_DEF2("_CAPI_LayerwiseBlockIfFused", "_CAPI_layerwise_block_if_fused",
              &Graph::LayerwiseBlockIfFused)
      GS_DEF2("_CAPI_QueueSampleLayers", "_CAPI_queue_sample_layers", &Graph::QueueSampleLayers)
      GS_DEF2("_CAPI_QueueSampleLayersBatched", "_CAPI_queue_sample_layers_batched",
              &Graph::QueueSampleLayersBatched)
      GS_DEF2("_CAPI_FusionSlicing", "_CAPI_fusion_slicing", &Graph::FusedBidirSlicing)
      GS_DEF2("_CAPI_BatchFusionSlicing", "_CAPI_batch_fusion_slicing",
              &Graph::BatchFusedBidirSlicing)
      GS_DEF2("_CAPI_BatchSlicing", "_CAPI_batch_slicing", &Graph::BatchSlicing)
      GS_DEF2("_CAPI_Split", "_CAPI_split", &Graph::Split)
      GS_DEF2("_CAPI_Decode", "_CAPI_decode", &Graph::Decode)
      GS_DEF2("_CAPI_GetBatchCOO", "GetBatchCOO", &Graph::GetBatchCOO)
      GS_DEF2("_CAPI_LoadCSC", "_CAPI_load_csc", &Graph::LoadCSC)
      GS_DEF2("_CAPI_LoadCSR", "_CAPI_load_csr", &Graph::LoadCSR)
      GS_DEF2("_CAPI_LoadCOO", "_CAPI_load_coo", &Graph::LoadCOO)
      GS_DEF2("_CAPI_LoadCSCWithColIds", "_CAPI_load_csc_with_col_ids", &Graph::LoadCSCWithColIds)
      GS_DEF2("_CAPI_AllValidNode", "_CAPI_all_valid_node", &Graph::AllValidNode)
      GS_DEF2("_CAPI_GetRows", "_CAPI_get_rows", &Graph::GetRows)
      GS_DEF2("_CAPI_GetCols", "_CAPI_get_cols", &Graph::GetCols)
      GS_DEF2("_CAPI_GetValidRows", "_CAPI_get_valid_rows", &Graph::GetValidRows)
      GS_DEF2("_CAPI_GetValidCols", "_CAPI_get_valid_cols", &Graph::GetValidCols)
      GS_DEF2("_CAPI_GetCOORows", "_CAPI_get_coo_rows", &Graph::GetCOORows)
      GS_DEF2("_CAPI_GetCooCols", "_CAPI_get_coo_cols", &Graph::GetCOOCols)
      GS_DEF2("_CAPI_Relabel", "_CAPI_relabel", &Graph::Relabel)
      GS_DEF2("_CAPI_Sum", "_CAPI_sum", &Graph::Sum)
      GS_DEF2("_CAPI_Normalize", "_CAPI_normalize", &Graph::Normalize)
      GS_DEF2("_CAPI_Divide", "_CAPI_divide", &Graph::Divide)
      GS_DEF2("_CAPI_EDivUSum", "_CAPI_e_div_u_sum", &Graph::EDivUSum)
      GS_DEF2("_CAPI_Metadata", "_CAPI_metadata", &Graph::MetaData)
      GS_DEF2("_CAPI_COOMetadata", "_CAPI_coo_metadata", &Graph::COOMetaData)
      GS_DEF2("_CAPI_CSCMetadata", "_CAPI_csc_metadata", &Graph::CSCMetaData)
      GS_DEF2("_CAPI_RandomWalk", "_CAPI_random_walk", &Graph::RandomWalk)
      GS_DEF2("_CAPI_SDDMM", "_CAPI_sddmm", &Graph::SDDMM)
      GS_DEF2("_CAPI_GetCSC", "_CAPI_get_csc", &Graph::GetCSCTensor)
      GS_DEF2("_CAPI_GetCSR", "_CAPI_get_csr", &Graph::GetCSRTensor)
      GS_DEF2("_CAPI_GetBatchCSC", "GetBatchCSC", &Graph::GetBatchCSC)
      GS_DEF2("_CAPI_GetCOO", "_CAPI_get_coo", &Graph::GetCOOTensor)
      GS_DEF2("_CAPI_SetCOO", "_CAPI_set_coo", &Graph::SetCOOByTensor)
      GS_DEF2("_CAPI_SetMetadata", "_CAPI_set_metadata", &Graph::SetMetaData)
      GS_DEF2("_CAPI_CSC2CSR", "_CAPI_csc2csr", &Graph::CSC2CSR)
      GS_DEF2("_CAPI_CSR2CSC", "_CAPI_csr2csc", &Graph::CSR2CSC)
      GS_DEF2("_CAPI_CSC2DCSR", "_CAPI_csc2dcsr", &Graph::CSC2DCSR)
      GS_DEF2("_CAPI_CSR2DCSC", "_CAPI_csr2dcsc", &Graph::CSR2DCSC)
      GS_DEF2("_CAPI_SetValidCols", "_CAPI_set_valid_cols", &Graph::SetValidCols)
      GS_DEF2("_CAPI_SetValidRows", "_CAPI_set_valid_rows", &Graph::SetValidRows)
      GS_DEF2("_CAPI_CreateSparseFormat", "_CAPI_create_sparse_format", &Graph::CreateSparseFormat);

  m.class_<HeteroGraph>("HeteroGraph")
      .def(torch::init<>())
      GS_DEF2("_CAPI_LoadFromHomo", "load_from_homo", &HeteroGraph::LoadFromHomo)
      GS_DEF2("_CAPI_GetHomoGraph", "get_homo_graph", &HeteroGraph::GetHomoGraph)
      GS_DEF2("_CAPI_MetapathRandomWalkFused", "metapath_random_walk_fused",
              &HeteroGraph::MetapathRandomWalkFused);
}

TORCH_LIBRARY(gs_ops, m) {
  m.def("_CAPI_ListSampling", &ListSampling);
  m.def("list_sampling", &ListSampling);
  m.def("_CAPI_ListSamplingWithProbs", &ListSamplingProbs);
  m.def("list_sampling_with_probs", &ListSamplingProbs);
  m.def("_CAPI_SplitByOffset", &SplitByOffset);
  m.def("SplitByOffset", &SplitByOffset);
  m.def("_CAPI_Unique", &UniqueOp);
  m.def("_CAPI_IndptrSplitByOffset", &IndptrSplitByOffset);
  m.def("IndptrSplitByOffset", &IndptrSplitByOffset);
  m.def("_CAPI_IndptrSplitBySize", &IndptrSplitBySize);
  m.def("IndptrSplitBySize", &IndptrSplitBySize);
  m.def("_CAPI_BatchCSRRelabel", &BatchCSRRelabel);
  m.def("BatchCSRRelabel", &BatchCSRRelabel);
  m.def("_CAPI_BatchCSRRelabelByKey", &BatchCSRRelabelByKey);
  m.def("BatchCSRRelabelByKey", &BatchCSRRelabelByKey);
  m.def("_CAPI_BatchCOORelabel", &BatchCOORelabel);
  m.def("BatchCOORelabel", &BatchCOORelabel);
  m.def("_CAPI_BatchCOORelabelByKey", &BatchCOORelabelByKey);
  m.def("BatchCOORelabelByKey", &BatchCOORelabelByKey);
  m.def("_CAPI_BatchConcat", &BatchConcat);
  m.def("BatchConcat", &BatchConcat);
  m.def("_CAPI_BatchSplit", &BatchSplit);
  m.def("BatchSplit", &BatchSplit);
  m.def("_CAPI_BatchUnique", &BatchUnique);
  m.def("BatchUnique", &BatchUnique);
  m.def("_CAPI_BatchUniqueByKey", &BatchUniqueByKey);
  m.def("BatchUniqueByKey", &BatchUniqueByKey);
  m.def("_CAPI_BatchUnique2", &BatchUnique2);
  m.def("BatchUnique2", &BatchUnique2);
  m.def("_CAPI_BatchUniqueByKey2", &BatchUniqueByKey2);
  m.def("BatchUniqueByKey2", &BatchUniqueByKey2);
  m.def("_CAPI_BatchEncode", &BatchEncode);
  m.def("BatchEncode", &BatchEncode);
  m.def("_CAPI_BatchDecode", &BatchDecode);
  m.def("BatchDecode", &BatchDecode);
  m.def("_CAPI_GetBatchOffsets", &GetBatchOffsets);
  m.def("GetBatchOffsets", &GetBatchOffsets);
  m.def("_CAPI_BatchCOOSlicing", &BatchCOOSlicing);
  m.def("BatchCOOSlicing", &BatchCOOSlicing);
  m.def("_CAPI_COORowSlicingGlobalId", &COORowSlicingGlobalId);
  m.def("COORowSlicingGlobalId", &COORowSlicingGlobalId);
  m.def("_CAPI_BatchListSamplingWithProbs", &BatchListSamplingProbs);
  m.def("batch_list_sampling_with_probs", &BatchListSamplingProbs);
  m.def("_CAPI_IndexSearch", &IndexSearch);
  m.def("index_search", &IndexSearch);
  // not in the reference: reproducible sampling (its seeds are compile-time constants)
  m.def("_CAPI_SetSeed", &SetSeed);
  m.def("_CAPI_SetThreadSeed", &SetThreadSeed);
  m.def("_CAPI_SampleBlocks", &SampleBlocks);
  m.def("_CAPI_SampleBlocksBatched", &SampleBlocksBatched);
  m.def("_CAPI_SetSampleAlgo", &SetSampleAlgo);
  // not in the reference: on = float sums of a COO-only graph add in edge order (same bits
  // every run) at the price of sorting its edges first
  m.def("_CAPI_SetOrderedSums", &SetOrderedSums);
  // not in the reference: off = _CAPI_SampleLayersBatched waits for every layer's edge count
  // before its relabel (buffers of the exact sizes) instead of queueing the relabel behind
  // the sampler
  m.def("_CAPI_SetBatchedNoWait", &SetBatchedNoWait);
  m.def("_CAPI_BatchedNoWaitCounts", &BatchedNoWaitCounts);
  // not in the reference: off = every sampling call settles its edge count before returning
  m.def("_CAPI_SetDeferredSampling", &SetDeferredSampling);
  // not in the reference: test hook for the recovery from a look-back that gave up
  m.def("_CAPI_DebugRaiseLookbackError", &DebugRaiseLookbackError);
}
