"""CPU oracle for the LIF fire path -- TEST INFRASTRUCTURE ONLY.

Only tests/, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import this
package.  The shipped package ``snn_gpu_training_bptt_amd`` never does.

* ``oracle.c_oracle``  -- ctypes binding of ``lif_oracle.c`` (scalar loops in the order of the
  reference's kernels, snnlib/cuda/snn_kernel_fp.cu:37-52 and snnlib/cuda/snn_kernel_bp.cu:117-138).
* ``oracle.gold_fire`` -- pure-PyTorch restatement of the reference's gold path
  (snnlib/example/gold_op.py:17-44); backward by autograd.
"""
