"""MI355X-native target-verify hot path of DFlash speculative decoding.

Host-side mirror of the dflash-mlx operators on this path (same names, argument
meaning and fallback behaviour), backed by hand-written gfx950 kernels in
``libdflash_mi355.so`` (C ABI: include/dflash_mi355.h):

* ``verify_matmul`` / ``verify_qmm`` - M=16 int4 affine quantized matmul;
  ``VerifyQuantizedLinear`` / ``install_verify_linears`` - the module swap.
* ``RecurrentRollbackCache`` / ``tape_replay_kernel`` - GatedDeltaNet tape-replay
  rollback; ``RollbackArena`` - the same for all layers in one launch;
  ``KVCache.trim`` - attention-cache trim.
* ``gated_delta_kernel_with_tape`` - the GatedDeltaNet forward that records the tape;
  ``gdn_layer`` - the layer call around it (fused glue kernels, pad-to-16 projections);
  ``loader`` - MLX-format 4-bit checkpoints; ``generate`` - the speculative cycle.
"""
__version__ = "0.1.0"
