"""CPU oracle for the GRPO logprob + loss hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``rl_amd/`` may import this package;
it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / reported CPU baseline.

Every function is a plain-PyTorch (CPU, fp32 unless stated) restatement of the
arithmetic of the reference implementation, cited per function as
``<reference file>:<lines>`` relative to the NeMo-RL source tree.  The
primitives the reference relies on (``log_softmax``, ``gather``, ``sort``,
``cumsum``, ``topk``, ``matmul``) are PyTorch's own, so torch on the CPU is
the legitimate ground truth for them.

Pinning status (what fixes each function besides its own text):

* ``logprob.*``            pinned: textbook ``log_softmax(x).gather`` identity,
                           autograd of that form, brute force on tiny vocab,
                           chunk == no-chunk, packed == per-sequence.
* ``sampling.*``           pinned by properties (outside top-k is -inf, kept
                           probabilities reach top_p, keep_mask == ~isinf) and
                           brute force.  PARITY UNPINNED for which of several
                           exactly tied values at the top-p boundary survives
                           (the reference sorts unstably); this oracle keeps
                           torch's stable ascending order.  Also unpinned: the
                           one boundary element of a row whose cumulative
                           probability there lies within fp32 rounding (about
                           1e-6) of 1 - top_p; softmax and cumsum sum in another
                           order on every device, the reference's included.
* ``loss.calculate_kl``    pinned: golden vectors of the reference's unit tests.
* ``loss.masked_mean``     pinned: closed form.
* ``loss.clipped_pg_loss`` pinned: closed-form losses of the reference's unit
                           tests (PPO clip, REINFORCE, on-policy, CISPO, KL,
                           IS/TIS/ICE-POP/seq-mask-tis, dual clip, GSPO).
                           PARITY UNPINNED for the diagnostics the reference
                           never tests numerically (token_mult_prob_error,
                           gen_kl_error, policy_kl_error, js_divergence_error,
                           sampling_importance_ratio, probs_ratio*): restated
                           from the source text and checked against
                           independent float64 formulas only.
* ``loss.sequence_packing_loss``  pinned: the identity the reference's own test
                           states (per-sequence wrapper == one loss call on the
                           unpacked batch, loss and gradient to 1e-5,
                           ``tests/unit/algorithms/test_sequence_packing_fusion.py:190-265``)
                           for additive metrics, and brute force for the
                           min / max merging (``tests/test_oracle_loss.py``).
* ``advantage.*``          pinned: golden vectors of the reference's unit tests.
* ``advantage.seq_logprob_error_masking``  pinned by brute-force loops on tiny
                           inputs (the reference's tests only mock it).
* ``logprob.logprobs_post_process``  pinned: ``log_softmax`` + ``gather``
                           identity and brute-force loops on tiny inputs.
* ``distill.*``            pinned: closed forms (uniform / one-hot rows, H(p,q) =
                           H(p) + KL; equal distributions give zero KL; a top-k
                           spanning the vocabulary gives the textbook KL), the
                           reference's stated backward formulas and brute force
                           (``tests/test_oracle_distill.py``).
* ``preference.*``         pinned: the closed-form cases of the reference's own
                           DPO tests (zero logits vs zero reference, SFT term of
                           the chosen rows, SFT-only == rescaled NLL) and a
                           loop-per-pair brute force
                           (``tests/test_oracle_preference.py``).
* ``lmhead.*``             pinned: forward == ``log_softmax(hidden @ W.T).gather``,
                           backward == torch autograd of that unfused form,
                           chunked == unchunked.  PARITY UNPINNED only for the
                           rounding of the reference's dW (accumulated per chunk
                           in the weights' dtype; the reference's one test of
                           this path needs Megatron, two GPUs and a model
                           download).
"""
