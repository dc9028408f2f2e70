"""CPU oracle for the speculative-decoding hot path.

TEST INFRASTRUCTURE ONLY.  These modules restate, in plain torch-on-CPU / numpy, what the
reference's own PyTorch path computes for one speculative cycle.  They exist so that the HIP
kernels can be checked against them; nothing that ships (the ``subspec_amd`` package and the
C-ABI library) imports, calls or links anything from here.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may use this package,
and only as the checker / the timed CPU baseline.

Every function cites the reference file:line it follows (paths relative to the reference root).

How each function is pinned (so a wrong sign / index / dropped term fails a test):

* ``verify.lossy_verify`` (prob gate)      – the 8 known-answer cases of the reference's
  ``tests/test_lossy_tree_verify.py`` (inputs + expected outputs + 7 diagnostics), kept as data in
  ``tests/golden/lossy_kat.json``.
* ``verify.lossy_verify`` (entropy gate, random 64-node trees, window 6, EOS, tie order) –
  golden vectors written by ``tests/golden/make_reference_vectors.py`` (imports the reference's pure-torch
  verifier in the build container only) + brute-force path enumeration on tiny trees +
  invariants (theta=0 entropy gate == exact verify).
* ``verify.exact_verify``                  – planted-path construction (answer known by design),
  equality with lossy(theta=0, entropy), golden vectors incl. ``skip_nodes`` > 0.
* ``topk.topk_expand``                     – ``torch.topk`` values bit-exact, brute force on tiny V,
  tie rule (value desc, flat index asc) by stable sort.
* ``tree`` helpers                         – brute-force ancestor closure; golden vectors for
  ``prune_to_depth`` / ``prune_to_top_n`` re-indexing.
* ``kv.compact``                           – closed-form gather; prefix/tail invariants.
* ``attention.tree_attention``             – ``F.scaled_dot_product_attention`` with the additive
  ``finfo.min`` mask over ``repeat_kv``-expanded heads (library routine) vs the explicit
  softmax(QK^T/sqrt d + M)V restatement.
* ``int4.linear``                          – closed form x @ ((Wq - z) * s).T; the special case
  s=1, z=0 reduces to an integer matmul.  The HQQ *quantizer* itself (hqq==0.2.6, absent) is
  **parity unpinned**: parity is defined on the linear given identical (Wq, scale, zero).
* ``decoder.decoder_layer``                – float32 restatement of the Qwen2 decoder layer the reference runs
  through HuggingFace; equals ``transformers``' own Qwen2 decoder (small random-weight model built in the
  test, called with a cached prefix, ``position_ids = prefix + depth`` and the additive ancestor mask, as
  ``_tree_decoding`` does) to 2e-4 in every layer's hidden state, the logits and the cached K / V rows;
  plus closed forms (rotary is a rotation, identity at position 0 and relative; zero output projections
  leave the residual stream; its attention block equals ``attention.tree_attention``).
* ``kv.compact_paged``                     – the reference's pool reorder restated literally
  (``compact_paged_reference``) for the identity page table; gather / compact / scatter equivalence for a
  permuted table.
* ``sampling``                             – Philox4x32-10 against Random123's known-answer vectors; the
  exponential race against a per-element loop and a chi-square test; the verifiers with pre-drawn target
  tokens against brute force and hand-built walks.  The random stream is this build's contract (torch's is
  not an interface); the distribution and the use of the draw are the reference's.
"""
