"""CPU oracle for the TorchGT sparse-attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` use it, and there only as the checker (or as the CPU
baseline being timed), never as the thing that produces a result.

Every function restates, in plain PyTorch / numpy, the algorithm of a reference
function and cites the reference file:line it follows.  The reference ships no
tests, fixtures or golden vectors, and it cannot be imported offline (it imports
torch_scatter / dgl / torch_geometric at module top), so each function is pinned
by independent checks in ``tests/test_oracle_*.py``:

=============================  ================================================
function                       pinned by
=============================  ================================================
sparse_attention               dense-softmax equivalence (torch.softmax), fp64
                               brute-force loops, closed-form special cases,
                               permutation / relabel invariants
sparse_attention (gradients)   torch autograd of the restatement; analytic
                               formulas checked by fp64 gradcheck
dense_bias_to_edge_bias        brute-force indexing loops
dense_attention                torch.softmax/matmul library routine with the
                               q*sqrt(d) quirk; brute-force loops; with a keep
                               mask: loops from the definition (softmax, mask /
                               (1 - p), times v) and the p = 0 reduction
graph_attn_bias                loops from the definition; torch's embedding for
                               the padding-index rows of the table gradients
fix_edge_index                 hand-computed known answer (N=3)
relabel_by_partition           hand-computed known answer
blockize / reformat_graph      hand-computed known answers (k=1, N=32, bs=16;
                               the compact-count misalignment after an empty
                               partition pair; the raw-edge branch of a sparse
                               tile) + structural invariants
build_csr                      numpy stable argsort + round-trip invariants
graph_attn_bias_multi_hop      reduces to graph_attn_bias (one hop, identity
                               hop matrices, adjacent pairs); fp64 loops from
                               the definition; halves when the distance doubles
gen_edge_input                 hand-computed known answer (path graph); every
                               row is a walk of existing edges from i to j of
                               the shortest length (scipy)
graph_node_feature             torch.nn.functional.embedding; hand-computed answer
graph-level graphormer_forward torch's layer_norm / linear / gelu / softmax
                               assembly; closed form without layers; node
                               relabelling and padding invariance
gt_forward (node-level GT)     torch's layer_norm / linear / relu / softmax on a
                               complete graph; closed form without layers;
                               commutes with node relabelling
nll_loss                       torch's CPU F.nll_loss (library routine); log C
                               for a uniform prediction
metis partition labels         PARITY UNPINNED: dgl/METIS is absent; partition
                               ids are always an explicit input here
=============================  ================================================
"""
