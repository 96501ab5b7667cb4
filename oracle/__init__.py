"""CPU oracle for the Monarch / KV-cache attention hot path.

THIS PACKAGE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker.  The product package never imports it and
raises when its HIP library is missing.

Every function restates (in own code: torch-CPU / numpy, float64 by default)
an algorithm of the reference and cites the reference file:line it follows.
What pins each function (so that a dropped term, a wrong index or a
transposed operand fails a test) is listed below; the checks themselves live
in ``tests/test_oracle_*.py``.

====================  ========================================================
function              pinned by
====================  ========================================================
blocks.to_blocks /    golden permutations of the reference's _get_rearrange_fns;
blocks.from_blocks    explicit index formula checked token by token, round
                      trip, identity-in-memory special case (f_tied=1,
                      w_reduce=1)
monarch.monarch_1iter golden vectors of the reference's monarch_attn_ref_op
                      (tests/golden/); b2=1 => dense softmax attention; b1=1,f=1 => dense;
                      implied N x N matrix L*R built with scalar loops has
                      unit row sums and reproduces the output; constant V;
                      permutation of KV block-frames; LSE merge of KV chunks;
                      Gibbs equality of the step-2 logit on the i==k diagonal
monarch.monarch_iter  golden vectors of the reference's own monarch_attn_slow for
                      num_iters in {1,2,3,8} (tests/golden/, <= 2e-6: the reference
                      runs its softmaxes in float32); num_iters=1 equals
                      monarch_1iter up to the 1/(1+1e-6) factor; b2=1 => dense
monarch.*_kv_cache,   compositions of the above with a cache write; pinned by
monarch.causal        slicing identities (causal == chunk by chunk)
dense.attention       torch.nn.functional.scaled_dot_product_attention (library
                      routine) and scalar loops on tiny inputs
prologue.rms_norm     torch.nn.functional.rms_norm; closed form
prologue.rope_*       closed form x*e^{i theta}; norm preservation; start_frame
                      shift == slicing a longer sequence; relative-position
                      property
cache.KVCacheState    hand-traced index sequences (7 chunks x 5 passes; a
                      window/sink eviction trace)
sched.*               closed form sigma(t); warped step list
====================  ========================================================
"""
