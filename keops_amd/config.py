"""Run-time knobs of the backend (counterpart of keopscore/keopscore/config: only the settings
that still mean something on ROCm are kept; CUDA discovery has no equivalent here).

Environment variables:
  KEOPS_AMD_CACHE     folder of the on-disk JIT cache (default: <package>/build)
  KEOPS_AMD_VERBOSE   "0" silences the informational messages
  KEOPS_HIP_ARCH      offload architecture used when no GPU is visible (default gfx950)
"""
import os
import sys

_PKG = os.path.dirname(os.path.abspath(__file__))

verbose = os.environ.get("KEOPS_AMD_VERBOSE", "1") != "0"

# chunked-mode thresholds, same values as keopscore/keopscore/config/chunks.py:19-35
dimchunk = 64
dim_treshold_chunk = 146
specdims_use_chunk = [99, 100, 102, 120, 133, 138, 139, 140, 141, 142]
dimfinalchunk = 64

# workgroup geometry of the tiled kernels
block_size = 256           # threads per workgroup (4 wavefronts)
max_rows_per_lane = int(os.environ.get("KEOPS_AMD_MAX_ROWS", 4))      # output rows held in the registers of one lane
lds_tile_bytes = 16384     # LDS bytes of one staged column tile
# block-sparse / batched launches: workgroups per compute unit that the choice of rows per lane keeps
irregular_wg_per_cu = int(os.environ.get("KEOPS_AMD_IRREGULAR_WG_PER_CU", 16))
# formula bodies of more than segment_threshold statements are cut into functions of segment_statements each
segment_threshold = int(os.environ.get("KEOPS_AMD_SEGMENT_MIN", 1024))
segment_statements = int(os.environ.get("KEOPS_AMD_SEGMENT", 512))
lse_group = int(os.environ.get("KEOPS_AMD_LSE_GROUP", 8))  # log-sum-exp: columns folded per running-maximum update

# matrix-core chunked scheme (csrc/kernels/keops_chunk_mfma.h): wavefronts (32 output rows each) per workgroup
chunk_waves = int(os.environ.get("KEOPS_AMD_CHUNK_WAVES", 8))
chunk_presplit = os.environ.get("KEOPS_AMD_CHUNK_PRESPLIT", "1") != "0"  # dense launches: pre-split copy of the weights
chunk_min_dim = int(os.environ.get("KEOPS_AMD_CHUNK_MIN_DIM", 24))    # smallest contraction served by the matrix-core chunked scheme
# squared distances below this fraction of |x|^2+|y|^2 are recomputed in float32 (0: never).  Default: 1/4, which
# bounds the relative error of every squared distance by 4 * 1.4e-7 (the expansion is off by about 1.4e-7 of the
# norms), the order of the rounding of the reference's own float32 sum; 1/8 below 32 components, where random pairs
# come that close often enough for the recomputation to cost more than it is worth (+50 % at D = 24)
# K-nearest-neighbour reductions with block-sparse ranges on the matrix-core scheme (0: the general-purpose ranges kernel)
knn_ranges = os.environ.get("KEOPS_AMD_KNN_RANGES", "1") != "0"
chunk_near = os.environ.get("KEOPS_AMD_CHUNK_NEAR", "auto")
# squared distances on the matrix cores: operand scale from the bulk of the rows when a few rows hold components far
# beyond the others', those rows (and rows with values that are not finite) computed pair by pair from the float32 data
chunk_robust = os.environ.get("KEOPS_AMD_CHUNK_ROBUST", "1") != "0"
# float64 contractions on the float64 matrix instruction (csrc/kernels/keops_chunk_f64.h)
chunk64 = os.environ.get("KEOPS_AMD_CHUNK64", "1") != "0"
chunk64_min_dim = int(os.environ.get("KEOPS_AMD_CHUNK64_MIN_DIM", 32))
chunk64_max_dim = 256          # the operands of 16 output rows fill 128 registers of a wavefront
chunk64_min_rows = int(os.environ.get("KEOPS_AMD_CHUNK64_MIN_ROWS", 4096))
chunk_max_dim = int(os.environ.get("KEOPS_AMD_CHUNK_MAX_DIM", 1024))  # largest contraction served by the matrix-core chunked scheme

# exponents of low-dimensional Gaussian kernel sums on the matrix cores (csrc/kernels/keops_radial_mfma.h)
radial = os.environ.get("KEOPS_AMD_RADIAL", "1") != "0"
radial_max_dim = 8                  # components of the points (7 D + 8 slots of the scalar product fit four instructions)
radial_max_dv = 8                   # components of the weights (16 accumulators per component in every lane)
# components of v up to which gradients with a factor <u_i, v_j> form it per pair in the matrix-core exponent kernels
# (dim(v) more fused multiply-adds per pair: 28.5 against 33.8 ms on the general-purpose kernel at 3 components,
# 45.3 against 42.5 ms at 8; 300 000 x 300 000 points in space)
radial_upair_max_dw = int(os.environ.get("KEOPS_AMD_RADIAL_UPAIR_MAX_DW", 5))
radial_bilinear = os.environ.get("KEOPS_AMD_RADIAL_BILINEAR", "1") != "0"   # a factor <u_i, v_j> out of the matrix cores, like the exponent
# ... up to this many components and k blocks of the slot vectors together (300 000 x 300 000 points in space, gradient
# with 8 weight components, five k blocks: 31.6 against 43.8 ms on the general-purpose kernel; 10 components, six k
# blocks: 64.8 against 49.8 ms)
radial_bilinear_max_dw = int(os.environ.get("KEOPS_AMD_RADIAL_BILINEAR_MAX_DW", 8))
radial_bilinear_max_nkb = int(os.environ.get("KEOPS_AMD_RADIAL_BILINEAR_MAX_NKB", 5))
radial_mm_max_dv = 32               # ... when the weighted sum runs on the matrix cores (the three terms of the weights in up to three blocks of 32 operand columns)
radial_rb2_max_dv = int(os.environ.get("KEOPS_AMD_RADIAL_RB2_MAX_DV", 4))  # two 32-row blocks per wavefront up to this many accumulated components
# columns per staged tile (multiple of 32); auto: 512, and 256 when the weighted sum runs on the matrix cores too (a tile
# change costs two barriers and the test of the tile's bound: 10^6 x 10^6 with one weight, 128 / 256 / 512 columns:
# 95.9 / 93.4 / 93.0 ms; gradient with respect to the points, 256 / 512 / 1024: 182.6 / 180.0 / 187.3 ms)
# accumulated components from which the weighted sum of the radial scheme runs on the matrix cores (per pair the vector
# ALU then issues v_exp_f32 and a three-term split instead of one fused multiply-add per component); 99: never
radial_mm_min_dv = int(os.environ.get("KEOPS_AMD_RADIAL_MM_MIN_DV", 7))
# bfloat16 terms of a kernel value in that product: 3 (24 bits: the float32 class) or 2 (both rounded to nearest:
# every kernel value is then off by up to 2^-17, 2.4e-6 rms, forty times the float32 rounding, which sums with
# cancellation do not forgive; 199 against 263 ms at eight components on 10^6 x 10^6 points, and the matrix cores
# then win from five components on: KEOPS_AMD_RADIAL_MM_MIN_DV=5)
radial_mm_terms = int(os.environ.get("KEOPS_AMD_RADIAL_MM_TERMS", 3))
radial_mm_rb = int(os.environ.get("KEOPS_AMD_RADIAL_MM_RB", 1))   # 32-row blocks per wavefront in that variant
radial_tile_j = os.environ.get("KEOPS_AMD_RADIAL_TJ", "auto")
# Dense launches decide per tile: a wavefront takes the exponents of a 32-column sub-tile from the matrix cores when
# |c| log2(e) (max |x^|^2 of its rows + max |y^|^2 of the sub-tile) <= this bound for the centred points (both clouds
# are sorted by that quantity); an exponent is off by at most 8 * 2^-24 of it, a kernel value by 3.3e-7 * limit <= 1e-5.
# The other sub-tiles are computed from exact differences in the same sweep.
radial_limit = float(os.environ.get("KEOPS_AMD_RADIAL_LIMIT", 30.0))
# ... unless more than this share of the pairs would be (estimated on the device from the sort's bucket counts): then
# the general-purpose kernel computes the whole sum
radial_exact_frac = float(os.environ.get("KEOPS_AMD_RADIAL_EXACT_FRAC", 0.25))
# block-sparse launches: one centre and one check per row range, |c| log2(e) (R_x^2 + min(R_y, R_x + reach)^2) <= this
radial_ranges_limit = float(os.environ.get("KEOPS_AMD_RADIAL_RANGES_LIMIT", 128.0))
radial_ranges = os.environ.get("KEOPS_AMD_RADIAL_RANGES", "1") != "0"  # block-sparse launches too (one centre per row range)
# calls below 2**29 pairs (23171 x 23171) stay on the general-purpose kernel: the sort, the per-tile maxima and the exact
# kernel around the sweep are a dozen small launches, 0.12 ms together.  Measured, matrix-core scheme against the
# general-purpose kernel: 16000^2 0.157 vs 0.103 ms, 23000^2 0.186 vs 0.174, 32000^2 0.252 vs 0.293, 50000^2 0.43 vs 0.64,
# 100000^2 1.19 vs 2.47 ms.  Batches and block-sparse launches (their pre-pass is another one): from 2**28 pairs on
radial_min_pairs_log2 = int(os.environ.get("KEOPS_AMD_RADIAL_MIN_PAIRS", 30))
radial_ranges_min_pairs_log2 = int(os.environ.get("KEOPS_AMD_RADIAL_RANGES_MIN_PAIRS", 29))

# matrix-core final-product scheme (csrc/kernels/keops_final_mfma.h): Sum_j f(x_i,y_j) * v_j with dim(v) large
final_chunk_min_dim = int(os.environ.get("KEOPS_AMD_FINAL_MIN_DIM", 24))   # smallest dim(v) that selects the scheme
final_max_blocks = int(os.environ.get("KEOPS_AMD_FINAL_NB", 8))            # 32-column accumulator tiles per wavefront
final_waves = int(os.environ.get("KEOPS_AMD_FINAL_WAVES", 8))              # wavefronts (32 output rows each) per workgroup
final_tile_j = int(os.environ.get("KEOPS_AMD_FINAL_TJ", 32))               # reduced rows per staged tile (even)
final_split3 = os.environ.get("KEOPS_AMD_FINAL_SPLIT3", "1") != "0"          # product in three bfloat16 terms per operand
# ... of the staged vectors and of the per-pair weights; 2: the weights in two terms, both rounded to nearest (off by up
# to 2^-17 each, 2.4e-6 rms: not the float32 class; C5b 68.8 against 70.6 ms, softmax_d64 4.70 against 5.09 ms)
final_weight_terms = int(os.environ.get("KEOPS_AMD_FINAL_WEIGHT_TERMS", 3))
final_period = int(os.environ.get("KEOPS_AMD_FINAL_PERIOD", 16384))        # block-sum period in reduced rows
# ... when the sums are kept in double (dtype_acc = float64, Kahan scheme): 64 matrix-instruction accumulations per fold
final_period_acc64 = int(os.environ.get("KEOPS_AMD_FINAL_PERIOD_ACC64", 1024))

# matrix-core KNN kernel (csrc/kernels/keops_knn_mfma.h)
knn_min_dim = int(os.environ.get("KEOPS_AMD_KNN_MIN_DIM", 2))         # smallest vector dimension served by the matrix-core KNN scheme
knn_tile_j = int(os.environ.get("KEOPS_AMD_KNN_TJ", 128))          # reference rows per LDS tile (<= 256)
knn_filter_tile_j = int(os.environ.get("KEOPS_AMD_KNN_FTJ", 256))  # reference rows per LDS tile of the fixed-threshold filter
knn_max_waves = int(os.environ.get("KEOPS_AMD_KNN_WAVES", 8))     # wavefronts per workgroup sharing one staged tile
knn_filter_waves = int(os.environ.get("KEOPS_AMD_KNN_FWAVES", 16))  # fixed-threshold filter: wavefronts per workgroup
knn_filter_qsets = int(os.environ.get("KEOPS_AMD_KNN_FQSETS", 2))   # and 32-query operand sets per wavefront
knn_sample = int(os.environ.get("KEOPS_AMD_KNN_SAMPLE", 16))            # sampling pass: every 16th reference
knn_sample_waves = int(os.environ.get("KEOPS_AMD_KNN_SWAVES", 8))  # sampling pass: wavefronts per workgroup
knn_sample_qsets = int(os.environ.get("KEOPS_AMD_KNN_SQSETS", 1))   # and 32-query operand sets per wavefront
vchunk_min_dim = int(os.environ.get("KEOPS_AMD_VCHUNK_MIN_DIM", 100))   # long elementwise sums beyond this many components keep their rows in memory
min_as_kmin = int(os.environ.get("KEOPS_AMD_MIN_AS_KMIN", 1))        # Min / ArgMin of SqDist on the KNN schemes (K = 1)
knn_highdim_margin = int(os.environ.get("KEOPS_AMD_KNN_HD_MARGIN", 6))   # extra approximate candidates kept per row by the high-dimensional KNN sweep
knn_min_work = int(os.environ.get("KEOPS_AMD_KNN_MIN_WORK", 1 << 32))      # smallest pairs x max(D, 16) served by the matrix-core KNN scheme
knn_batch_max = int(os.environ.get("KEOPS_AMD_KNN_BATCH_MAX", 64))    # batched KNN: at most this many batches are served one by one
knn_batch_min_work = int(os.environ.get("KEOPS_AMD_KNN_BATCH_MIN_WORK", 1 << 33))  # ... of at least this many pairs x max(D, 8) each
knn_lds_budget = 150 * 1024                                        # LDS bytes a KNN workgroup may use (160 KB per CU)
knn_i8 = os.environ.get("KEOPS_AMD_KNN_I8", "1") != "0"           # fixed-threshold filter on signed bytes (v_mfma_i32_32x32x32_i8) when its slack allows
knn_qsets = int(os.environ.get("KEOPS_AMD_KNN_QSETS", 1))          # 32-query operand sets per wavefront (<= 2)


_build_folder = None


def get_build_folder():
    folder = _build_folder or os.environ.get("KEOPS_AMD_CACHE") or os.path.join(_PKG, "build")
    os.makedirs(folder, exist_ok=True)
    return folder


def set_build_folder(path=None):
    """Folder of the on-disk cache of compiled kernel modules; None restores the default."""
    global _build_folder
    _build_folder = None if path is None else os.path.abspath(path)
    return get_build_folder()


def message(*args, **kwargs):
    # progress messages go to stderr: stdout belongs to the caller (bench.py prints one JSON line there)
    if verbose:
        kwargs.setdefault("file", sys.stderr)
        print("[keops_amd]", *args, **kwargs)
