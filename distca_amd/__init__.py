"""MI355X-native core-attention (CA) server kernels behind DistCA's call surface.

  ops              a2a_memcpy_non_cp / a2a_memcpy_cp / pre_a2a_grad_acc   (shard pack/unpack)
  dispatch         pre/post_a2a_* compositions and the [out|lse], [dO|O|lse|q] token layouts
  fused_comm_attn  ca_varlen_fwd / ca_varlen_bwd, _qkv_to_attn_out_fwd/_bwd, the server tick
  scheduler        host mirror of the on-device tile scheduler
  workloads        synthetic task batches of the benchmark configurations

Everything computes through libdistca_ca.so (HIP, gfx950); importing the package does not
load it, the first op call does and raises if it is missing.
"""
__version__ = "0.1.0"
