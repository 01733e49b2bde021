// A C++ caller of the host layer: compiles against graph.h / graph_ops.h / tensor_ops.h /
// hetero_graph.h exactly as a C++ user of the reference would (its tests/*.cc include "graph.h"
// and call gs::Graph with int64 CUDA tensors), links libgs.so, and checks each operator of the
// sampling path against a closed form.  Exit code 0 and a last line "ALL OK" when everything holds.
//
// Built by graph_sampling_amd/build.py (build_cpp_check); run on a GPU by tests/test_gpu_cpp_api.py.
#include <torch/torch.h>

#include <cstdio>
#include <string>
#include <vector>

#include "graph.h"
#include "graph_ops.h"
#include "hetero_graph.h"
#include "tensor_ops.h"

using gs::_COO;
using gs::_CSC;
using gs::_CSR;
using torch::Tensor;

static int g_failed = 0, g_checked = 0;
#define CHECK_THAT(cond)                                                   \
  do {                                                                     \
    ++g_checked;                                                           \
    if (!(cond)) {                                                         \
      ++g_failed;                                                          \
      std::printf("FAILED %s:%d  %s\n", __FILE__, __LINE__, #cond);        \
      std::fflush(stdout);                                                 \
    }                                                                      \
  } while (0)

static torch::TensorOptions I64() { return torch::TensorOptions().dtype(torch::kInt64).device(torch::kCUDA); }
static torch::TensorOptions F32() { return torch::TensorOptions().dtype(torch::kFloat32).device(torch::kCUDA); }
static Tensor ids(std::vector<int64_t> v) { return torch::tensor(v, torch::kInt64).to(torch::kCUDA); }

// `cols` columns of `deg` edges each; edge j of column c points at row c * deg + j
static c10::intrusive_ptr<gs::Graph> BandGraph(int64_t cols, int64_t deg) {
  auto g = c10::make_intrusive<gs::Graph>(false);
  g->LoadCSC(torch::arange(0, cols + 1, I64()) * deg, torch::arange(0, cols * deg, I64()));
  return g;
}

static void ColumnSlices() {
  std::puts("column slices"); std::fflush(stdout);
  auto g = BandGraph(20, 5);
  Tensor pick = ids({7, 2, 2, 19});
  auto sub = g->Slicing(pick, 0, _CSC, _CSC);
  auto csc = sub->GetCSC();
  CHECK_THAT(csc->indptr.equal(torch::arange(0, 5, I64()) * 5));
  Tensor want = (pick.unsqueeze(1) * 5 + torch::arange(0, 5, I64()).unsqueeze(0)).reshape({-1});
  CHECK_THAT(csc->indices.equal(want));
  CHECK_THAT(sub->GetNumCols() == 4 && sub->GetNumEdges() == 20);
  CHECK_THAT(sub->GetCols().equal(pick));

  // the format-level function under the method: offsets, edge -> column, ids, positions in the parent
  auto tmp = gs::CSCColSlicing(g->GetCSC(), pick, true);
  CHECK_THAT(tmp.first->indptr.equal(csc->indptr));
  CHECK_THAT(tmp.first->coo_in_indices.equal(want));
  CHECK_THAT(tmp.first->coo_in_indptr.equal(torch::arange(0, 4, I64()).repeat_interleave(5)));
  CHECK_THAT(tmp.second.equal(want));  // row id == position in this graph

  // induced subgraph in one call == column slice then row slice
  Tensor both = torch::arange(3, 9, I64());
  auto two_steps = g->Slicing(both, 0, _CSC, _CSC)->Slicing(both, 1, _CSC, _CSC);
  auto one_step = g->FusedBidirSlicing(both, both);
  CHECK_THAT(two_steps->GetCSC()->indptr.equal(one_step->GetCSC()->indptr));
  CHECK_THAT(two_steps->GetCSC()->indices.equal(one_step->GetCSC()->indices));
}

static void UniformSampling() {
  std::puts("uniform sampling"); std::fflush(stdout);
  auto g = BandGraph(20, 5);
  // a fanout of at least the degree keeps every edge, in order
  auto all = g->Sampling(0, 5, false, _CSC, _CSC);
  CHECK_THAT(all->GetCSC()->indptr.equal(g->GetCSC()->indptr));
  CHECK_THAT(all->GetCSC()->indices.equal(g->GetCSC()->indices));
  // below the degree: `fanout` distinct edges of the column
  auto three = g->Sampling(0, 3, false, _CSC, _CSC);
  CHECK_THAT(three->GetCSC()->indptr.equal(torch::arange(0, 21, I64()) * 3));
  Tensor picked = three->GetCSC()->indices.reshape({20, 3});
  CHECK_THAT((picked.floor_divide(5) == torch::arange(0, 20, I64()).unsqueeze(1)).all().item<bool>());
  Tensor sorted = std::get<0>(picked.sort(1));
  CHECK_THAT((sorted.slice(1, 1, 3) != sorted.slice(1, 0, 2)).all().item<bool>());
  // with replacement every non-empty column gets exactly `fanout` edges
  auto many = g->Sampling(0, 8, true, _CSC, _CSC);
  CHECK_THAT(many->GetCSC()->indptr.equal(torch::arange(0, 21, I64()) * 8));
  CHECK_THAT((many->GetCSC()->indices.reshape({20, 8}).floor_divide(5) ==
              torch::arange(0, 20, I64()).unsqueeze(1)).all().item<bool>());

  // slice and sample in one call
  Tensor seeds = ids({4, 0, 11});
  auto fused = g->ColumnwiseFusedSlicingAndSampling(seeds, 5, false);
  CHECK_THAT(fused->GetCSC()->indptr.equal(torch::arange(0, 4, I64()) * 5));
  CHECK_THAT(fused->GetCSC()->indices.equal(
      (seeds.unsqueeze(1) * 5 + torch::arange(0, 5, I64()).unsqueeze(0)).reshape({-1})));
  auto fused2 = g->ColumnwiseFusedSlicingAndSampling(seeds, 2, false);
  CHECK_THAT(fused2->GetNumEdges() == 6);
  CHECK_THAT((fused2->GetCSC()->indices.reshape({3, 2}).floor_divide(5) == seeds.unsqueeze(1)).all().item<bool>());
}

static void WeightedSampling() {
  std::puts("weighted sampling"); std::fflush(stdout);
  auto g = BandGraph(6, 8);
  // one overwhelming weight per column: that edge is always among the picks
  Tensor w = torch::full({48}, 1e-9f, F32());
  Tensor heavy = torch::arange(0, 6, I64()) * 8 + ids({3, 0, 7, 5, 1, 2});
  w.index_put_({heavy}, 1.0f);
  auto sub = g->SamplingProbs(0, w, 2, false, _CSC, _CSC);
  CHECK_THAT(sub->GetCSC()->indptr.equal(torch::arange(0, 7, I64()) * 2));
  Tensor picked = sub->GetCSC()->indices.reshape({6, 2});
  CHECK_THAT((picked == heavy.unsqueeze(1)).any(1).all().item<bool>());
  CHECK_THAT((picked.select(1, 0) != picked.select(1, 1)).all().item<bool>());
}

static void RelabelAndNodes() {
  std::puts("relabel, node queries"); std::fflush(stdout);
  // 3 columns named 10, 11, 12 whose edges point at rows 40, 10, 41 | 41 | 12, 40
  auto g = c10::make_intrusive<gs::Graph>(true);
  g->LoadCSCWithColIds(ids({10, 11, 12}), ids({0, 3, 4, 6}), ids({40, 10, 41, 41, 12, 40}));
  auto r = g->Relabel();
  CHECK_THAT(std::get<0>(r).equal(ids({10, 11, 12, 40, 41})));  // columns first, then rows as met
  CHECK_THAT(std::get<1>(r) == 5 && std::get<2>(r) == 3);
  CHECK_THAT(std::get<3>(r).equal(ids({0, 3, 4, 6})));
  CHECK_THAT(std::get<4>(r).equal(ids({3, 0, 4, 4, 2, 3})));
  CHECK_THAT(std::get<6>(r) == "csc");
  CHECK_THAT(g->AllValidNode().equal(ids({10, 11, 12, 40, 41})));
  CHECK_THAT(g->GetValidRows().equal(ids({10, 12, 40, 41})));

  CHECK_THAT(gs::TensorUnique(ids({9, 4, 9, 1, 4, 7})).equal(ids({9, 4, 1, 7})));
  auto br = gs::BatchTensorRelabel({ids({5, 3}), ids({8, 3, 6})}, {ids({6, 5, 8, 3}), ids({2})});
  CHECK_THAT(std::get<0>(br).equal(ids({5, 3, 8, 6})));
  CHECK_THAT(std::get<1>(br)[0].equal(ids({3, 0, 2, 1})));
  CHECK_THAT(std::get<1>(br)[1].equal(ids({-1})));

  // a column slice that renames its rows on the way
  auto band = BandGraph(20, 5);
  auto renamed = band->Slicing(ids({3, 1}), 0, _CSC, _COO, true);
  CHECK_THAT(renamed->GetRows().equal(ids({15, 16, 17, 18, 19, 5, 6, 7, 8, 9})));
  CHECK_THAT(renamed->GetCOO()->row.equal(torch::arange(0, 10, I64())));
  CHECK_THAT(renamed->GetCOO()->col.equal(ids({0, 0, 0, 0, 0, 1, 1, 1, 1, 1})));
}

static void Formats() {
  std::puts("format conversions"); std::fflush(stdout);
  // columns 0..3 with rows {2,0} {} {1,2,0} {1}; LoadCSC takes the matrix as square, so 4 rows
  auto g = c10::make_intrusive<gs::Graph>(false);
  g->LoadCSC(ids({0, 2, 2, 5, 6}), ids({2, 0, 1, 2, 0, 1}));
  g->CSC2CSR();
  auto csr = g->GetCSR();
  CHECK_THAT(csr->indptr.equal(ids({0, 2, 4, 6, 6})));
  CHECK_THAT(csr->indices.equal(ids({0, 2, 2, 3, 0, 2})));      // stable: edges of a row keep their order
  CHECK_THAT(csr->e_ids.value().equal(ids({1, 4, 2, 5, 0, 3})));
  auto coo = gs::GraphCSC2COO(g->GetCSC(), true);
  CHECK_THAT(coo->row.equal(ids({2, 0, 1, 2, 0, 1})));
  CHECK_THAT(coo->col.equal(ids({0, 0, 2, 2, 2, 3})));
  auto back = gs::GraphCOO2CSC(coo, 4, true);
  CHECK_THAT(back->indptr.equal(ids({0, 2, 2, 5, 6})) && back->indices.equal(ids({2, 0, 1, 2, 0, 1})));
  // rows kept by a row slice are renamed to their position in the request
  auto rows = g->Slicing(ids({2, 0}), 1, _CSC, _CSC);
  CHECK_THAT(rows->GetCSC()->indptr.equal(ids({0, 2, 2, 4, 4})));
  CHECK_THAT(rows->GetCSC()->indices.equal(ids({0, 1, 0, 1})));
}

static void EdgeData() {
  std::puts("sums, normalise, divide, SDDMM"); std::fflush(stdout);
  auto g = c10::make_intrusive<gs::Graph>(false);
  g->LoadCSC(ids({0, 2, 2, 5, 6}), ids({2, 0, 1, 2, 0, 1}));
  Tensor w = torch::tensor({1.f, 2.f, 3.f, 4.f, 5.f, 6.f}).to(torch::kCUDA);
  g->SetData(w);
  CHECK_THAT(torch::allclose(g->Sum(0, 1, _CSC), torch::tensor({3.f, 0.f, 12.f, 6.f}).to(torch::kCUDA)));
  CHECK_THAT(torch::allclose(g->Sum(0, 2, _CSC), torch::tensor({5.f, 0.f, 50.f, 36.f}).to(torch::kCUDA)));
  CHECK_THAT(torch::allclose(g->Sum(1, 1, _CSR), torch::tensor({7.f, 9.f, 5.f, 0.f}).to(torch::kCUDA)));
  CHECK_THAT(torch::allclose(g->Sum(1, 1, _COO), torch::tensor({7.f, 9.f, 5.f, 0.f}).to(torch::kCUDA)));
  auto n = g->Normalize(0, _CSC);
  CHECK_THAT(torch::allclose(n->GetData().value(),
                             torch::tensor({1 / 3.f, 2 / 3.f, 3 / 12.f, 4 / 12.f, 5 / 12.f, 1.f}).to(torch::kCUDA)));
  auto d = g->Divide(torch::tensor({2.f, 1.f, 4.f, 3.f}).to(torch::kCUDA), 0, _CSC);
  CHECK_THAT(torch::allclose(d->GetData().value(),
                             torch::tensor({.5f, 1.f, .75f, 1.f, 1.25f, 2.f}).to(torch::kCUDA)));

  // out[e] = lhs[row of e] + rhs[col of e], two features wide, on two formats
  Tensor lhs = torch::arange(0, 8, F32()).reshape({4, 2});
  Tensor rhs = torch::arange(0, 8, F32()).reshape({4, 2}) * 10;
  Tensor row = ids({2, 0, 1, 2, 0, 1}), col = ids({0, 0, 2, 2, 2, 3});
  Tensor want = lhs.index({row}) + rhs.index({col});
  for (int64_t fmt : {_COO, _CSC}) {
    Tensor out = torch::zeros({6, 2}, F32());
    g->SDDMM("add", lhs, rhs, out, 0, 2, fmt);
    CHECK_THAT(torch::allclose(out, want));
  }
  Tensor dots = torch::zeros({6, 1}, F32());
  Tensor rhs3 = torch::arange(0, 8, F32()).reshape({4, 2});
  g->SDDMM("dot", lhs, rhs3, dots, 0, 2, _CSC);
  CHECK_THAT(torch::allclose(dots.reshape({-1}), (lhs.index({row}) * rhs3.index({col})).sum(1)));
}

static void Lists() {
  std::puts("list sampling"); std::fflush(stdout);
  Tensor data = torch::arange(100, 164, I64());
  auto all = gs::ListSampling(data, 64, false);
  CHECK_THAT(std::get<0>(all).equal(data) && std::get<1>(all).equal(torch::arange(0, 64, I64())));
  auto ten = gs::ListSampling(data, 10, false);
  CHECK_THAT(std::get<0>(ten).numel() == 10);
  CHECK_THAT(std::get<0>(ten).equal(data.index({std::get<1>(ten)})));
  CHECK_THAT(std::get<0>(at::_unique(std::get<1>(ten))).numel() == 10);
  Tensor p = torch::zeros({64}, F32());
  p.index_put_({ids({5, 17, 40})}, 1.0f);
  auto weighted = gs::ListSamplingProbs(data, p, 3, false);  // items of weight zero are never taken
  CHECK_THAT(std::get<0>(std::get<1>(weighted).sort()).equal(ids({5, 17, 40})));
}

static void Walks() {
  std::puts("walks"); std::fflush(stdout);
  // a ring: the only neighbour of node c is (c + 1) % 8
  auto ring = c10::make_intrusive<gs::Graph>(false);
  ring->LoadCSC(torch::arange(0, 9, I64()), (torch::arange(0, 8, I64()) + 1) % 8);
  Tensor trace = ring->RandomWalk(ids({0, 5}), 3);
  CHECK_THAT(trace.size(0) == 2 && trace.size(1) == 4);
  // the memory is step-major: [step][walker]
  CHECK_THAT(trace.reshape({-1}).equal(ids({0, 5, 1, 6, 2, 7, 3, 0})));

  // two relations: "up" sends node c to c + 1 (none from 3), "stay" keeps c
  auto up = c10::make_intrusive<gs::Graph>(false);
  up->LoadCSC(ids({0, 1, 2, 3, 3}), ids({1, 2, 3}));
  auto stay = c10::make_intrusive<gs::Graph>(false);
  stay->LoadCSC(torch::arange(0, 5, I64()), torch::arange(0, 4, I64()));
  gs::HeteroGraph h;
  h.LoadFromHomo({"n"}, {{"n", "up", "n"}, {"n", "stay", "n"}}, {up, stay});
  Tensor t = h.MetapathRandomWalkFused(ids({0, 2}), {"up", "stay", "up", "up"});
  // walker 0: 0 1 1 2 3; walker 1: 2 3 3 -1 -1 (stuck walkers stay at -1)
  CHECK_THAT(t.reshape({-1}).equal(ids({0, 2, 1, 3, 1, 3, 2, -1, 3, -1})));
  CHECK_THAT(h.GetHomoGraph("up")->GetNumEdges() == 3);
}

int main() {
  if (!torch::cuda::is_available()) {
    std::puts("no GPU: nothing was run");
    return 2;
  }
  ColumnSlices();
  UniformSampling();
  WeightedSampling();
  RelabelAndNodes();
  Formats();
  EdgeData();
  Lists();
  Walks();
  std::printf("%d checks, %d failed\n", g_checked, g_failed);
  if (g_failed == 0) std::puts("ALL OK");
  return g_failed ? 1 : 0;
}
