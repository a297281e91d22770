"""Which kernel the size rules pick for every BASELINE configuration, pinned on the CPU (the query functions are plain
integer arithmetic when the number of compute units is passed in). A change of a rule that moves a configuration onto
another kernel has to show up here, next to the GPU parity test that covers that kernel:
  1D kernels (numbering of turbofno_set_1d_algo): 1 SIMT, 2 / 3 matrix cores with 512- / 256-thread blocks, 4 matrix
  cores with 32-channel output tiles, 5 one wavefront per item, 6 K split over the waves of a block, 7 K split over a
  cluster of blocks (only with an exchange buffer attached), 8 tiles of 128 output channels;
  2D algorithms: 1 three kernels (X axis first), 2 whole image, 3 three kernels (rows first).
GPU parity of each: tests/test_gpu_parity.py (every selector forced), tests/test_gpu_fullsize.py (the configurations at
full size), tests/test_gpu_cluster.py (7), tests/test_gpu_large_grids.py."""
import turbofno_amd as tf

CUS = 256       # MI355X


def test_1d_kernel_of_configuration_1():
    assert tf.query_1d_kernel(128, 1, 64, 8, CUS) == 4


def test_1d_kernels_of_configuration_2():
    # 112 problems, all of them at most one block per CU: matrix cores, eight waves per block, 32-channel output tiles
    for bs in (1, 2, 4, 8, 16, 32, 64):
        for DY in (128, 256):
            for N in (64, 128):
                for K in (8, 16, 24, 32):
                    assert tf.query_1d_kernel(DY, bs, N, K, CUS) == 4, (bs, DY, N, K)


def test_1d_kernels_of_configuration_3():
    for K in (64, 128):
        assert tf.query_1d_kernel(256, 64, 128, K, CUS, exchange_attached=True) == 7
        assert tf.query_1d_kernel(256, 64, 128, K, CUS, exchange_attached=False) == 6


def test_2d_algorithms_of_configurations_4_and_5():
    for D in (128, 256):
        for K in (16, 32):
            assert tf.query_2d_algo(1, D, D, K, 64) == tf.ALGO_THREE_KERNEL
            assert tf.query_2d_algo(4, D, D, K, 64) == tf.ALGO_THREE_KERNEL
            assert tf.query_2d_algo(16, D, D, K, 64) == tf.ALGO_WHOLE_IMAGE
    assert tf.query_2d_algo(16, 256, 256, 64, 64) == tf.ALGO_WHOLE_IMAGE          # the headline problem


def test_large_grids_and_long_axes():
    # the reference's own benchmark regime: thousands of signals per channel
    assert tf.query_1d_kernel(256, 4096, 64, 64, CUS) == 3
    assert tf.query_1d_kernel(256, 4096, 128, 64, CUS) == 8
    assert tf.query_1d_kernel(128, 4096, 64, 64, CUS) == 5
    assert tf.query_1d_kernel(128, 4096, 128, 128, CUS) == 8
    assert tf.query_1d_kernel(512, 4096, 64, 32, CUS) == 1
    # axes above 256, small problems: three stages, the longer axis (or, for squares with enough images, the contiguous
    # one) first
    assert tf.query_2d_algo(2, 512, 512, 64, 64) == tf.ALGO_ROWS_FIRST
    assert tf.query_2d_algo(1, 512, 512, 32, 64) == tf.ALGO_THREE_KERNEL
    assert tf.query_2d_algo(8, 256, 1024, 32, 64) == tf.ALGO_ROWS_FIRST
    assert tf.query_2d_algo(4, 1024, 256, 32, 64) == tf.ALGO_THREE_KERNEL
    assert tf.query_2d_algo(2, 1024, 1024, 32, 64) == tf.ALGO_ROWS_FIRST
    # large ones: the whole-image kernels (512 / 1024 rows as interleaved parts of 256, long rows with 32 / 64 lanes),
    # from a volume of input and output that depends on the lengths
    assert tf.query_2d_algo(16, 512, 512, 32, 64) == tf.ALGO_WHOLE_IMAGE
    assert tf.query_2d_algo(4, 512, 512, 32, 64) == tf.ALGO_WHOLE_IMAGE            # 768 MiB
    assert tf.query_2d_algo(4, 512, 512, 16, 64) == tf.ALGO_THREE_KERNEL           # 640 MiB
    assert tf.query_2d_algo(16, 512, 256, 32, 64) == tf.ALGO_WHOLE_IMAGE
    assert tf.query_2d_algo(4, 512, 256, 32, 64) == tf.ALGO_THREE_KERNEL           # 384 MiB
    assert tf.query_2d_algo(16, 512, 128, 32, 64) == tf.ALGO_WHOLE_IMAGE
    assert tf.query_2d_algo(8, 512, 128, 32, 64) == tf.ALGO_THREE_KERNEL
    assert tf.query_2d_algo(16, 256, 512, 32, 64) == tf.ALGO_WHOLE_IMAGE
    assert tf.query_2d_algo(8, 1024, 256, 32, 64) == tf.ALGO_WHOLE_IMAGE           # 1536 MiB
    assert tf.query_2d_algo(4, 1024, 256, 32, 64) == tf.ALGO_THREE_KERNEL          # 768 MiB
    assert tf.query_2d_algo(16, 256, 1024, 32, 64) == tf.ALGO_WHOLE_IMAGE          # 3072 MiB
    assert tf.query_2d_algo(8, 256, 1024, 32, 64) == tf.ALGO_ROWS_FIRST            # 1536 MiB
    assert tf.query_2d_algo(16, 1024, 1024, 32, 64) == tf.ALGO_WHOLE_IMAGE
    assert tf.query_2d_algo(4, 1024, 1024, 32, 64) == tf.ALGO_ROWS_FIRST           # 3072 MiB


def test_queries_answer_zero_for_arguments_the_calls_refuse():
    assert tf.query_1d_kernel(256, 4, 64, 12, CUS) == 0             # K not a multiple of 8
    assert tf.query_1d_kernel(2048, 4, 64, 8, CUS) == 0             # no kernel of that length
    assert tf.query_1d_kernel(200, 4, 64, 8, CUS) == 0              # not a power of two
    assert tf.query_2d_algo(1, 200, 256, 16, 64) == 0
    assert tf.query_2d_algo(1, 2048, 512, 16, 64, tf.ALGO_WHOLE_IMAGE) == 0
    assert tf.query_2d_algo(1, 256, 256, 16, 60) == 0
    assert tf.query_2d_algo(1, 256, 256, 16, 64, 9) == 0
    # an explicit algorithm is returned as it is
    assert tf.query_2d_algo(1, 256, 256, 16, 64, tf.ALGO_WHOLE_IMAGE) == tf.ALGO_WHOLE_IMAGE
    assert tf.query_2d_algo(1, 512, 1024, 16, 64, tf.ALGO_WHOLE_IMAGE) == tf.ALGO_WHOLE_IMAGE
