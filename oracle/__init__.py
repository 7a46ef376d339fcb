"""CPU restatement of RetroInfer's wave-index path (reference: wennitao/RetrievalAttention).

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the product: it is the
checker that tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py compare the
HIP kernels against.  The product (retrievalattention_amd/) never imports it.

Every function cites the reference file:line it follows.  The 16-bit element type (bfloat16 or IEEE
half, the two the reference runs in) is taken from the inputs: roundings go to that type.  The reference stores no golden vectors
for this path; tests/golden/known_answers.json holds hand-worked known answers for every part below
(initial tokens, a clustering followed by hand, softmax cases in closed form, ties and masked clusters
in the selection, the buffer cut-off, a block cache trace, rational attention results), derived in
tests/golden/make_known_answers.py without this package.  How each function is pinned:

  scoring.batch_gemm_softmax      the reference's own test oracle bmm -> /sqrt(d) -> softmax
                                  (library/retroinfer/test/test_batch_gemm_softmax.py:9-18, atol 1e-3)
  scoring.select                  torch.sum / masked_fill_ / topk are library routines; checked
                                  against torch.topk value-for-value and against brute force
  copies.*                        the loop oracles of library/retroinfer/test/test_gather_copy.py
                                  (:110-127, :190-194, :233-237), bit-exact
  wavebuf.LruModel                the reference's own BufferManager, compiled from its source by
                                  oracle/build_ref.py into oracle/_ref/ (tests/test_wavebuf_ref.py:
                                  same hit/miss/update lists step by step, block id values aside);
                                  a hand-followed trace; invariants (hit <=> resident, capacity,
                                  unique block ids, least-recently-touched eviction)
  wavebuf.DeviceLruModel          the device-side block cache manager's arithmetic (recency as a step
                                  stamp plus the order inside the step, victims by (stamp, order)):
                                  the same policy as LruModel, pinned to it over random multi-probe
                                  traces (hit/miss lists, residency and eviction order; block id
                                  values aside) and by the same invariants
  kmeans.*                        brute force on tiny inputs in fp64, plus invariants (partition of
                                  the tokens, centroid*size = sum of keys, empty cluster keeps its
                                  centroid, float32 init formula, remainder tokens); the fixed
                                  summation order of kmeans.cluster_sums (blocks of 256 tokens) by a
                                  plain-loop restatement
  pipeline.decode_step            composition of the above; with zone_logits, next-layer cluster
                                  estimation (zones from a predicted query, retroinfer_cache.py:582-617)
  attention.weighted_flash_decoding   PARITY UNPINNED against the reference: the callee
                                  (github.com/Starmys/flash-attention, branch "weighted") is not in
                                  the reference tree and has no test there.  Semantics are inferred
                                  from the call sites (cache_hub/retroinfer_cache.py:611-617,
                                  :666-674) and pinned only by closed forms: w = 1 reduces to
                                  softmax attention (torch SDPA); merging with a previous partial
                                  equals attention over the concatenated keys; one token per
                                  cluster makes the estimate exact; identical keys in a cluster
                                  make the estimate exact for any sizes.
"""
