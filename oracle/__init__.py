"""CPU oracle for the Evoformer hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in ``fastfold_amd`` may import this package;
it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / timed CPU baseline.

``oracle.evoformer_ref``  plain-PyTorch fp32 restatement of the reference's
                          ``fastfold.model.nn`` Evoformer (block, stack and all
                          sub-modules, nn-layout parameter names), extra-MSA stack,
                          template pair stack and point-wise attention, input and recycling
                          embedders.
``oracle.ops_np``         float64 numpy restatements of the op-level kernels
                          (fused softmax, LayerNorm, attention core, the three
                          elementwise fusions, tri-mul / OPM contractions).
"""
