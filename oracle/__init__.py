"""CPU oracle for the JVP flash-attention hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package (``jvp_flash_attention_amd``) may import this
package.  Its only callers are ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``, and they use it as the checker, never as
the thing measured or shipped.

Three independent statements of the same mathematics live here:

``sdpa_jvp``   the reference's *own* test oracle: PyTorch math SDPA under
               forward-mode AD (reference ``tests/test_jvp_attention.py:548-561``
               and ``:595-597``), extended with ``autograd.grad`` through the
               tangent, which the reference never tests.
``dense``      closed-form dense numpy fp64 formulas for O, O', M, mu and every
               gradient (no autograd involved).
``tiled``      a restatement of the reference's tile loop (online softmax with
               running max / sum / tangent statistics, reference
               ``jvp_flash_attention/jvp_attention.py:125-336``, ``:862-933``,
               ``:1010-1033``) and of its backward recomputation
               (``:1384-1411``, ``:1415-1707``), plus the tangent-path backward
               the reference lacks.

``dropout``    the keep pattern of the library's dropout (a hash of seed and entry index) in numpy; ``dense`` takes
               the resulting matrix as ``keep_scale``.

Pinning (what each function is checked against in ``tests/test_oracle.py``):

* ``dense.forward`` / ``dense.backward`` vs ``sdpa_jvp`` (library routine) in
  fp64 for no mask / causal / boolean key padding / additive bias;
* ``dense.forward`` tangent vs central finite differences of the primal;
* ``dense.backward`` vs a brute-force finite-difference gradient of the scalar
  loss on tiny inputs (catches a dropped term or a wrong sign independently of
  autograd);
* invariants: rows of P' sum to zero (constant V, V'=0 gives O'=0), O' is
  linear in the tangents, the gT=0 backward reduces to the reference's
  first-order backward formulas (``jvp_attention.py:1541-1553``, ``:1687-1697``);
* ``dense`` with ``keep_scale`` vs torch's softmax times a fixed matrix under ``torch.func.jvp`` and
  ``autograd.grad`` (SDPA's definition of dropout written out), all mask modes; ``dropout`` vs the bijectivity
  and statistics the mix must have on the CPU, and bit for bit vs the pattern the library exports on the GPU;
* ``tiled`` vs ``dense`` for every tile size that divides L and for ragged L.

Parity unpinned by the reference itself: the tangent-path gradients
(d<gT,O'>/d{q,k,v,q',k',v'}) do not exist in the reference
(``jvp_attention.py:2831`` takes ``do, _``; ``:2976-2978`` returns ``None`` for
the tangent slots), so only the SDPA library route, finite differences and the
closed form pin them.  The reference's own deviations from SDPA for float masks
(``:247-251`` scales the mask by sm_scale; ``:1519-1522`` drops the bias in the
backward) are deliberately not reproduced: the oracle follows SDPA semantics.
"""
