"""CPU oracle for the paged / quantized KV-cache attention path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``areno_amd/`` may import this package;
it is the checker that the HIP kernels are compared against (tests, the smoke
entry point and the CPU-baseline leg of the benchmark), never a fallback.

Four restatements live here:

* ``block_table_ref`` -- the page lists of the scheduler state (free list, per-sequence pages,
  padded tables, prefill slots; ``areno/engine/data/rollout_state.py:55-56,128-151,212-225,282-285``,
  ``areno/engine/inference.py:573-580,651-658``).
* ``rope_ref`` -- the layer's steps in front of the path: per-head RMSNorm
  (``areno/accel/csrc/normalization.cu:34-56``) and rotary embedding
  (``areno/engine/layers/rotary.py:17-52``) with the eager ops' roundings.
* ``attention_ref`` / ``quant_ref`` -- PyTorch (CPU) restatement of the
  reference's pure-PyTorch attention (``areno/accel/attention.py:25-76``), of
  its cache stores (``areno/engine/layers/attention_backend/infer.py:245-288``)
  and of this build's own quantizer closed forms.
* ``native_kernels.c`` (+ ``native.py`` ctypes wrapper) -- plain-C restatement of
  the reference's CUDA kernels' algorithm (``areno/accel/csrc/attention.cu``:
  update l.526-553, split l.555-654, reduce l.656-702, varlen l.145-242),
  including the per-key online-softmax recurrence and the empty-split rule.

How each function is pinned (none of them by retyping its own formula):

=========================  ====================================================
function                   pinned by (tests/test_oracle_cpu.py)
=========================  ====================================================
ref_attention              float64 triple-loop brute force; torch SDPA with an
                           explicit mask; window=None == window>=L; window=0
ref_paged_decode           block-permutation / NaN-padding invariance, GQA ==
                           MHA on repeat_interleave'd KV, L=0 -> out == v_new,
                           equal keys -> mean(V); agrees with native C split/
                           reduce restatement for num_splits in {1,2,8,64}
ref_varlen / paged prefill per-sequence SDPA; ctx=0 == varlen; n=1 == decode
ref_cache_write / update   snapshot diff: exactly the addressed rows change
quantize_int8              numpy float64 brute force of the closed form; error
                           bound |x - x^| <= s/2; absmax -> +-127; zero rows
quantize_fp8               exhaustive 256-entry decode table built from the
                           OCP e4m3fn bit layout; torch's own CPU cast
ref_rmsnorm                float64 restatement; unit-RMS output for w = 1,
                           scale invariance rmsnorm(c x) == rmsnorm(x)
ref_rope                   position 0 is the identity; pair norms preserved;
                           rope(p1) then rope(p2) == rope(p1 + p2) in float64;
                           complex-multiplication form x * exp(i p w)
RefBlockTables             the values the reference's scheduler test holds
                           (tests/test_inference_scheduler_cpu.py:110-156
                           there); every page free or owned exactly once;
                           FIFO hand-out and give-back order
                           (tests/test_block_table_oracle_cpu.py)
=========================  ====================================================

The reference repository holds no golden vectors, known-answer tests or
fixtures for the attention kernels (its 27 test files are CPU-only and never
execute them), so there is nothing of the reference's to replay there; the reference's
Python was read, not imported.  The CUDA sources cannot be compiled here (no
nvcc), so there is no ``oracle/_ref`` build.
"""
