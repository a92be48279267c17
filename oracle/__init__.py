"""CPU restatement of the reference's Winograd / DWM convolution algorithm.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may use it, and there only as the
checker, never as the thing measured or shipped.

Modules
-------
cook_toom   exact-rational Cook-Toom generator + the literal F(2,r) tables
            (reference: wincnn.py:7-70, matrix_conv.py:12-40, matrix_convnd.py:14-27)
split_plan  DWM kernel split rule (reference: src/base_conv_launchers.h:58-388,
            src/base_conv_launchers.cu:307-313)
tiles       wino_split / wino_concat index maps
            (reference: Split_and_Concat.py:4-82, src/split_and_concat_kernels.cu:8-129)
winograd    filter / input / output transforms, batched product, the
            matrix_conv-style pipeline and the native DWM pipeline
            (reference: matrix_conv.py:137-254, matrix_conv3d.py:139-290,
            src/split_kernel.cu:14-203, src/winograd_conv.cpp:17-127, dwm.py:5-145)

Pinning status (what independent facts each function is checked against lives
in tests/test_oracle_*.py):
  cook_toom.*          pinned: literal tables in the reference source (F(2,1..3),
                       commented F(2,5) and F(2,9)), exact rational FIR identity,
                       textbook F(4,3) matrices, and - for the whole-kernel tiles
                       F(2,4..7) and F(9,5), fractional points included - the output
                       of the reference's own generator, kept as exact rationals in
                       tests/golden/cook_toom_reference_tables.json (written once by
                       tests/golden/make_cook_toom_tables.py).
  split_plan.*         pinned: all 36 keys of the reference LUT (golden JSON).
  tiles.*              pinned: torch unfold / brute-force loops, odd edges.
  winograd.*           pinned: fp64 torch conv2d/conv3d, integer-exact KATs,
                       the reference kernels' unrolled spot formulas.  The stacked
                       form of dwm_conv (pieces added by the batched product, which
                       the reference does not do) is pinned by the same fp64
                       convolution and integer-exact checks; so is the form with
                       pieces of two taps (split_plan.axis_pairs, dwm_conv(stacked=2)),
                       a split the reference does not use either.
  Tables F(2,8..11) of the reference (matrix_conv.py:36-39) are not restated:
  nothing here uses them.
"""
