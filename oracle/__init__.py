"""CPU oracle for the picotron hot path.  TEST INFRASTRUCTURE ONLY.

Everything under ``oracle/`` is a plain-torch restatement (fp32 / fp64, runs on the
host) of the algorithms in the reference's ``picotron/context_parallel/context_parallel.py``
and ``picotron/model.py``.  It exists to check the HIP kernels and to be timed as the
reported CPU baseline.  Nothing in the shipped package ``picotron_amd`` imports it;
only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg do.

Parity status of each oracle function (what pins it, see ``tests/test_oracle_*.py``):

* ``ring.block_forward``      pinned: fp64 ``softmax``/``logsumexp`` closed form, ``F.scaled_dot_product_attention``
* ``ring.block_backward``     pinned: ``torch.autograd.grad`` through the closed form, ``gradcheck``
* ``ring.merge``              pinned: ``torch.logaddexp`` + exp-weighted mean, identity/commutativity invariants
* ``ring.schedule`` & friends pinned: brute force against full-sequence causal attention for every rank, W <= 8
* ``ring.rope_slice`` / ``ring.position_ids`` / ``ring.causal_mask``  pinned: integer closed forms (exact)
* ``layers.get_cos_sin``      pinned: fp64 closed form, transformers' ``LlamaRotaryEmbedding``
* ``layers.apply_rotary_pos_emb`` pinned: transformers' ``apply_rotary_pos_emb``; rotation invariants
* ``layers.rmsnorm*``         pinned: transformers' ``LlamaRMSNorm``, ``F.rms_norm``, autograd
* ``layers.swiglu*``          pinned: ``F.silu`` (library), autograd
* ``layers.cross_entropy*``   pinned: ``F.cross_entropy`` (library), autograd
* ``optim.adamw_step`` / ``master_step`` pinned: ``torch.optim.AdamW`` step by step
* ``optim.lp_step``           pinned: torch's fused AdamW on bf16 parameters (rounding points of the stored values)
* ``model.OracleLlama`` / ``model.train_step``  pinned: transformers' ``LlamaForCausalLM`` with the same weights (logits,
                              loss, every gradient, one AdamW step), MHA and GQA, with and without the ring
                              (``tests/test_oracle_model.py``)

The reference ships no golden vectors for any of these functions.
"""
