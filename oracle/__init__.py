"""CPU oracle for the InfLLM streaming memory-attention path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the product:
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker (or as the timed CPU
baseline), never as a compute path of ``infllm_amd``.

The modules restate, in fp32 torch on the CPU, the algorithm of the reference's
torch path:

* ``oracle.rope``        <- inf_llm/attention/rope.py:4-112
* ``oracle.multistage``  <- inf_llm/attention/dot_production_attention/torch_impl.py:6-96
                            and base.py:3-30
* ``oracle.stream``      <- inf_llm/attention/context_manager.py:196-816 (stateful,
                            window-relative cursors like the reference)
* ``oracle.absolute``    <- the same path re-derived in absolute stream positions
                            (brute force over the whole stream; used to pin
                            ``oracle.stream``'s index arithmetic)

Pinning status (the reference ships no tests, fixtures or golden vectors for
this path, so every pin below is mathematical; see tests/test_oracle_*.py):

* rope:        fp64 complex rotation, norm/identity/relative-position invariants.
* multistage:  equals one dense softmax over the concatenated masked logits
               (torch.softmax / F.scaled_dot_product_attention) and pure-Python
               loops on tiny shapes; row sums of probabilities are 1.
* stream:      cross-checked against ``oracle.absolute`` (independent derivation),
               closed forms for init/unit boundaries and unit counts, invariance
               under how a stream is cut into append() calls, reduction to causal
               SDPA with standard RoPE when the stream fits the local window.
* cache model: policy never changes results; pure-Python dict/stable-sort model.

What stays "parity unpinned": the reference's exact bf16 rounding sequence and
``torch.topk`` tie order (both outside the stated acceptance: fp32 reference,
ties within 1e-3 relative excluded).
"""
