"""CPU oracle for the quantized routed-expert matmul path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``tensorfold_amd/`` may import this package; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` use it, and only as the checker.

It restates, on the CPU, the arithmetic the reference defines for the path:

* ``affine``  - MLX 4-bit affine format, dequant-then-matmul, expert epilogue rounding points
                (families/qwen3_5/cuda/qmm.py:132-149, families/qwen3_5/cuda/reference.py:11-15,
                cuda/experts.cuh:53-103, cuda/moe.py:131-142)
* ``routing`` - per-row top-k with softmax-over-selected weights and the stable pair sort into items
                (cuda/moe.py:58-85, cuda/experts.cu:157-285, tests/cuda/test_experts.py:107-115)
* ``exl3``    - EXL3 codebooks, circular bitstream, tile permutation, Hadamard-128 layer
                (cuda/exl3/format.py:31-180, docs/recipes/exl3.md:43-74)
* ``orc.c``   - a plain-C second statement of the integer parts (nibble order, bit-by-bit trellis decode) and an
                OpenMP dequant-then-matmul used as the timed CPU baseline (``native.py`` binds it with ctypes)

How each function is pinned (none is "parity unpinned"):
  nibble order / dequant  : one-hot identity reads back every nibble (tests/cuda/test_qmm.py:98-111), hand-built
                            word 0x76543210, numpy vs C vs pure-Python loops
  dequant-then-matmul     : float64 textbook GEMV on tiny inputs
  epilogues               : closed forms at chosen points (relu^2, SwiGLU with and without clip) in float64
  top-k ids               : brute-force sort by (-logit, id); all-equal logits -> ids 0..k-1
                            (tests/cuda/test_nemotron_kernels.py:71-80)
  routing weights         : scipy softmax over the selected logits
  plan                    : quadratic brute force; 37 rows on one expert -> items 16, 16, 5
                            (tests/cuda/test_experts.py:91-104)
  EXL3 codebooks          : hand-computed values from the prose spec, Python big-int + struct('e') decoder,
                            0.5 < std < 2 (tests/test_exl3_format.py:63-72)
  EXL3 bitstream          : vectorised numpy decoder vs C bit-by-bit vs pure-Python bit-by-bit, all 27 combos;
                            E(256) = 256 * bits (tests/test_exl3_format.py:87-96)
  tile permutation        : bijection onto 16 x 16 (tests/test_exl3_format.py:100-101)
  packed signs            : KAT [0b1000000000000101, 0] -> -1 at {0, 2, 15} (tests/test_exl3_format.py:129-134)
  Hadamard / layer        : Sylvester recursion == (-1)^popcount(i & j); (H/sqrt 128)^2 = I;
                            x @ dequantize == forward to 1e-12 (tests/test_exl3_format.py:113-126)
"""
