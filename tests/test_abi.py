"""CPU-side checks of the C-ABI boundary: the shared library loads without a GPU, exports
every symbol include/of3pair.h declares, and rejects bad arguments with the documented status
codes before any kernel would be launched.  No compute call is made here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "of3pair.h")


@pytest.fixture(scope="module")
def lib():
    from of3pair import _lib
    from of3pair import build as of3_build

    if not of3_build.is_built():
        of3_build.build()
    return _lib.load()


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(of3_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = _declared_symbols()
    for required in ("of3_trimul_fwd", "of3_trimul_proj", "of3_trimul_contract", "of3_trimul_out",
                     "of3_triattn_fwd", "of3_triattn_proj", "of3_triattn_flash", "of3_triattn_out",
                     "of3_version", "of3_last_hip_error", "of3_status_string", "of3_padded_n",
                     "of3_trimul_contract_variant",
                     "of3_trimul_workspace_bytes", "of3_triattn_workspace_bytes",
                     "of3_trimul_workspace_bytes_for", "of3_triattn_workspace_bytes_for",
                     "of3_transition_fwd", "of3_pair_bias_fwd", "of3_layer_norm_fwd", "of3_template_tail_fwd",
                     "of3_attn_pair_bias_fwd", "of3_attn_pair_bias_workspace_bytes", "of3_transition_rows_fwd",
                     "of3_transition_rows_workspace_bytes", "of3_attn_pair_bias_workspace_bytes_for",
                     "of3_transition_rows_workspace_bytes_for"):
        assert required in names


def test_library_exports_every_declared_symbol(lib):
    from of3pair import _lib

    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared_symbols():
        assert hasattr(raw, name), "libof3pair.so does not export %s" % name
        assert name in _lib.SIGNATURES, "ctypes binding lacks %s" % name
    assert sorted(_lib.SIGNATURES) == _declared_symbols()


def test_version_and_status_strings(lib):
    assert lib.of3_version() >= 1
    assert lib.of3_status_string(0) == b"ok"
    assert b"workspace" in lib.of3_status_string(-2)
    assert b"invalid" in lib.of3_status_string(-1)


def test_padded_n(lib):
    assert lib.of3_padded_n(1) == 128
    assert lib.of3_padded_n(128) == 128
    assert lib.of3_padded_n(129) == 256
    assert lib.of3_padded_n(768) == 768
    assert lib.of3_padded_n(0) == 0


def test_workspace_sizes(lib):
    n, np_ = 768, 768
    assert lib.of3_trimul_workspace_bytes(1, n, 128, 128) == 3 * 128 * np_ * np_ * 2
    qkv = n * 4 * np_ * 32 * 2
    want = 3 * qkv + 4 * n * np_ * 4 + n * np_ * 4 + n * n * 128 * 2
    assert lib.of3_triattn_workspace_bytes(1, n, 128, 4, 32) == want
    # unsupported shapes are reported as OF3_EINVAL (-1)
    assert lib.of3_trimul_workspace_bytes(1, n, 128, 64) == -1
    assert lib.of3_trimul_workspace_bytes(1, n, 96, 96) == -1
    assert lib.of3_triattn_workspace_bytes(1, n, 128, 8, 16) == -1
    assert lib.of3_triattn_workspace_bytes(1, 0, 128, 4, 32) == -1


FAKE = 0x10000  # non-null, 256-byte aligned, never dereferenced: validation fails first


def _s3(a, b, c):
    from of3pair import _lib

    return _lib.strides3((a, b, c))


def test_trimul_fwd_rejects_bad_arguments(lib):
    from of3pair import _lib

    zs = _s3(64 * 64 * 128, 64 * 128, 128)
    ptrs = [FAKE] * 10
    ws_need = lib.of3_trimul_workspace_bytes(1, 64, 128, 128)

    def call(z=FAKE, strides=zs, B=1, N=64, C=128, CH=128, ws=FAKE, ws_bytes=ws_need, dtype=_lib.OF3_DTYPE_BF16):
        return lib.of3_trimul_fwd(z, strides, None, None, *ptrs, FAKE, B, N, C, CH, 1, 0, ws, ws_bytes, dtype, None)

    assert call(dtype=7) == _lib.OF3_EINVAL                        # unknown dtype code
    # fp32 has its own (larger) workspace and looser shape rules; never call it with a workable argument set here
    need32 = lib.of3_trimul_workspace_bytes_for(_lib.OF3_DTYPE_F32, 1, 64, 128, 128)
    # a and b in three bf16 terms (12 bytes per element pair, more than 2 fp32 arrays), x, the weights split in three
    assert need32 == 12 * 128 * 64 * 64 + 128 * 64 * 64 * 4 + 6 * 6 * 128 * 128
    assert call(dtype=_lib.OF3_DTYPE_F32, ws_bytes=need32 - 1) == _lib.OF3_ENOSPC
    assert call(dtype=_lib.OF3_DTYPE_F32, C=300, CH=300) == _lib.OF3_EINVAL
    assert call(dtype=_lib.OF3_DTYPE_F32, z=FAKE + 2, ws_bytes=need32) == _lib.OF3_EINVAL
    assert call(C=96, CH=96) == _lib.OF3_EINVAL                   # unsupported channel count
    assert call(N=0) == _lib.OF3_EINVAL
    assert call(ws=None) == _lib.OF3_EINVAL                        # null workspace
    assert call(ws=FAKE + 8) == _lib.OF3_EINVAL                    # misaligned workspace
    assert call(ws_bytes=ws_need - 1) == _lib.OF3_ENOSPC          # workspace too small
    assert call(z=None) == _lib.OF3_EINVAL                         # null tensor
    assert call(z=FAKE + 2) == _lib.OF3_EINVAL                     # misaligned tensor
    assert call(strides=_s3(64 * 64 * 128, 64 * 128 + 4, 128)) == _lib.OF3_EINVAL  # stride not a multiple of 8


def test_triattn_fwd_rejects_bad_arguments(lib):
    from of3pair import _lib

    xs = _s3(64 * 64 * 128, 64 * 128, 128)
    ptrs = [FAKE] * 8
    ws_need = lib.of3_triattn_workspace_bytes(1, 64, 128, 4, 32)

    def call(x=FAKE, B=1, N=64, C=128, H=4, D=32, ws=FAKE, ws_bytes=ws_need, dtype=_lib.OF3_DTYPE_BF16):
        return lib.of3_triattn_fwd(x, xs, None, None, *ptrs, FAKE, B, N, C, H, D, 1e9, 0, ws, ws_bytes, dtype, None)

    assert call(dtype=7) == _lib.OF3_EINVAL
    need32 = lib.of3_triattn_workspace_bytes_for(_lib.OF3_DTYPE_F32, 1, 64, 128, 4, 32)
    # q, k, v in three bf16 terms (18 bytes per element, more than 3 fp32 arrays), o, the triangle bias, the split weights
    assert need32 == 18 * 64 * 4 * 64 * 32 + 64 * 64 * 128 * 4 + 4 * 64 * 64 * 4 + 6 * 5 * 128 * 128
    assert call(dtype=_lib.OF3_DTYPE_F32, ws_bytes=need32 - 1) == _lib.OF3_ENOSPC
    assert call(dtype=_lib.OF3_DTYPE_F32, D=72, ws_bytes=need32) == _lib.OF3_EINVAL  # head width beyond 64
    assert call(H=8) == _lib.OF3_EINVAL
    assert call(D=64) == _lib.OF3_EINVAL
    assert call(ws_bytes=ws_need - 1) == _lib.OF3_ENOSPC
    assert call(x=None) == _lib.OF3_EINVAL


def test_stage_entry_points_validate(lib):
    from of3pair import _lib

    assert lib.of3_trimul_contract(None, FAKE, FAKE, 1, 64, 128, 0, None) == _lib.OF3_EINVAL
    assert lib.of3_trimul_contract(FAKE, FAKE, FAKE, 1, 64, 128, 9, None) == _lib.OF3_EINVAL   # unknown variant
    assert lib.of3_trimul_contract(FAKE, FAKE, FAKE, 1, 64, 96, 0, None) == _lib.OF3_EINVAL    # unsupported CH
    assert lib.of3_triattn_flash(FAKE, FAKE, FAKE, FAKE, FAKE, None, 1, 64, 4, 32, None) == _lib.OF3_EINVAL


def test_shapes_beyond_32_bit_position_counts_are_refused(lib):
    """B * NP * NP must fit a 32-bit integer (the kernels count positions and tiles in int): larger
    shapes return OF3_EINVAL before any launch, in the stage entry points as in the fused ones."""
    from of3pair import _lib

    big_n, big_b = 46464, 40000  # 46464^2 > 2^31 ; 40000 * 256^2 > 2^31
    assert lib.of3_trimul_contract(FAKE, FAKE, FAKE, 1, big_n, 128, 0, None) == _lib.OF3_EINVAL
    assert lib.of3_trimul_contract(FAKE, FAKE, FAKE, big_b, 256, 128, 0, None) == _lib.OF3_EINVAL
    assert lib.of3_triattn_flash(FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 1, big_n, 4, 32, None) == _lib.OF3_EINVAL
    assert lib.of3_triattn_flash(FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, big_b, 256, 4, 32, None) == _lib.OF3_EINVAL
    assert lib.of3_trimul_workspace_bytes(1, big_n, 128, 128) == _lib.OF3_EINVAL
    assert lib.of3_triattn_workspace_bytes(big_b, 256, 128, 4, 32) == _lib.OF3_EINVAL
    assert lib.of3_trimul_workspace_bytes_for(_lib.OF3_DTYPE_F32, big_b, 256, 128, 128) == _lib.OF3_EINVAL
    assert lib.of3_trimul_contract_variant(1, big_n, 128) == _lib.OF3_EINVAL
    # the largest shapes that pass are still accepted by the size queries
    assert lib.of3_trimul_workspace_bytes(1, 46336, 128, 128) > 0
    assert lib.of3_trimul_contract_variant(1, 768, 128) in (1, 2, 3, 4)
    assert lib.of3_trimul_contract_variant(1, 768, 96) == _lib.OF3_EINVAL


def test_contract_variant_choice_follows_the_measured_table(lib):
    """Tile variant per token count on 256 compute units (the count the library assumes without a device):
    at each of these sizes the choice is the variant that was fastest inside the block on an MI355X
    (1: 256 x 192, 2: 256 x 128, 3: 256 x 256, 4: 384 x 192 tiles)."""
    measured_best = {256: 2, 320: 4, 448: 3, 512: 3, 576: 4, 640: 4, 700: 4, 768: 4, 769: 3, 800: 3, 850: 3,
                     900: 3, 960: 3, 1000: 3, 1100: 4, 1280: 3, 2048: 3}
    got = {n: lib.of3_trimul_contract_variant(1, n, 128) for n in measured_best}
    assert got == measured_best
    assert lib.of3_trimul_contract_variant(4, 512, 64) == 3  # the template stack: 256 planes of 512 x 512


def test_check_maps_status_to_exceptions(lib):
    from of3pair import _lib

    _lib.check(0, "ok")
    with pytest.raises(ValueError):
        _lib.check(_lib.OF3_EINVAL, "x")
    with pytest.raises(RuntimeError):
        _lib.check(_lib.OF3_ENOSPC, "x")


def test_template_entry_points_validate(lib):
    """Argument checks run before any device work: bad shapes and null pointers are refused."""
    from of3pair import _lib as L

    p = 256  # any non-null, 16-byte aligned value: it is never dereferenced on these paths
    assert lib.of3_layer_norm_fwd(None, p, p, p, 8, 64, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL
    assert lib.of3_layer_norm_fwd(p, p, p, p, 0, 64, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL
    assert lib.of3_layer_norm_fwd(p, p, p, p, 8, 96, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL
    assert lib.of3_layer_norm_fwd(p, p, p, p, 8, 300, L.OF3_DTYPE_F32, None) == L.OF3_EINVAL
    assert lib.of3_layer_norm_fwd(p + 2, p, p, p, 8, 64, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL
    assert lib.of3_template_tail_fwd(p, p, p, p, p, 1, 0, 16, 64, 128, 1, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL
    assert lib.of3_template_tail_fwd(p, p, p, p, p, 1, 2, 16, 32, 128, 1, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL
    assert lib.of3_template_tail_fwd(p, p, p, p, p, 1, 2, 16, 64, 64, 1, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL
    assert lib.of3_template_tail_fwd(p, None, p, p, p, 1, 2, 16, 64, 128, 1, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL
    assert lib.of3_template_tail_fwd(p, p, p, None, p, 1, 2, 16, 64, 128, 0, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL
    assert lib.of3_template_tail_fwd(p, p, p, p, p, 1, 2, 16, 64, 128, 1, 7, None) == L.OF3_EINVAL


def test_attn_pair_bias_entry_point_validates(lib):
    from of3pair import _lib as L

    assert lib.of3_attn_pair_bias_workspace_bytes(1, 768, 384, 16, 24) == 3 * 16 * 768 * 32 * 2 + 2 * 768 * 384 * 2
    assert lib.of3_attn_pair_bias_workspace_bytes(1, 768, 384, 24, 16) > 0
    for bad in ((1, 768, 256, 16, 16), (1, 768, 384, 16, 32), (1, 768, 384, 12, 32), (1, 768, 384, 32, 12), (0, 768, 384, 16, 24),
                (1, 1 << 17, 384, 16, 24)):
        assert lib.of3_attn_pair_bias_workspace_bytes(*bad) == L.OF3_EINVAL
    p = 256
    args = [p] * 2 + [None] + [p] * 9 + [1, 64, 384, 16, 24, 1e9, 0, p, 1 << 30]
    assert lib.of3_attn_pair_bias_fwd(*args, 7, None) == L.OF3_EINVAL                     # unknown dtype
    wide = list(args)
    wide[14] = 1024                                                                       # C_s beyond the fp32 kernels
    assert lib.of3_attn_pair_bias_fwd(*wide, L.OF3_DTYPE_F32, None) == L.OF3_EINVAL
    assert lib.of3_attn_pair_bias_workspace_bytes_for(L.OF3_DTYPE_F32, 2, 100, 384, 16, 24) == 5 * 2 * 100 * 384 * 4
    assert lib.of3_attn_pair_bias_workspace_bytes_for(L.OF3_DTYPE_BF16, 1, 768, 384, 16, 24) == \
        lib.of3_attn_pair_bias_workspace_bytes(1, 768, 384, 16, 24)
    assert lib.of3_attn_pair_bias_workspace_bytes_for(L.OF3_DTYPE_F32, 1, 100, 384, 4, 96) == L.OF3_EINVAL
    small = list(args)
    small[-1] = 1024
    assert lib.of3_attn_pair_bias_fwd(*small, L.OF3_DTYPE_BF16, None) == L.OF3_ENOSPC
    nul = list(args)
    nul[5] = None                                                                         # b_q missing
    assert lib.of3_attn_pair_bias_fwd(*nul, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL


def test_transition_rows_entry_point_validates(lib):
    from of3pair import _lib as L

    assert lib.of3_transition_rows_workspace_bytes(768, 384, 1536) == 768 * 1536 * 2
    for bad in ((0, 384, 1536), (768, 128, 512), (768, 384, 1000), (768, 384, 192)):
        assert lib.of3_transition_rows_workspace_bytes(*bad) == L.OF3_EINVAL
    p = 256
    args = [p, None] + [p] * 6 + [64, 384, 1536, 0, p, 1 << 30]
    assert lib.of3_transition_rows_fwd(*args, 7, None) == L.OF3_EINVAL
    wide = list(args)
    wide[10] = 4096                                                                       # hidden width beyond the fp32 kernel
    assert lib.of3_transition_rows_fwd(*wide, L.OF3_DTYPE_F32, None) == L.OF3_EINVAL
    assert lib.of3_transition_rows_workspace_bytes_for(L.OF3_DTYPE_F32, 768, 384, 1536) == 0
    assert lib.of3_transition_rows_workspace_bytes_for(L.OF3_DTYPE_F32, 768, 600, 1536) == L.OF3_EINVAL
    small = list(args)
    small[-1] = 16
    assert lib.of3_transition_rows_fwd(*small, L.OF3_DTYPE_BF16, None) == L.OF3_ENOSPC
    nul = list(args)
    nul[4] = None
    assert lib.of3_transition_rows_fwd(*nul, L.OF3_DTYPE_BF16, None) == L.OF3_EINVAL

def test_transition_workspace_variant_validates_on_the_host(lib):
    """of3_transition_fwd_ws: the fp32 workspace holds the weights split into three bf16 terms; bf16 needs none."""
    from of3pair import _lib as L

    assert lib.of3_transition_workspace_bytes_for(L.OF3_DTYPE_BF16, 1, 64, 128, 512) == 0
    need = lib.of3_transition_workspace_bytes_for(L.OF3_DTYPE_F32, 1, 64, 128, 512)
    assert need == 6 * 3 * 512 * 128
    assert lib.of3_transition_workspace_bytes_for(L.OF3_DTYPE_F32, 1, 64, 300, 512) == L.OF3_EINVAL
    assert lib.of3_transition_workspace_bytes_for(7, 1, 64, 128, 512) == L.OF3_EINVAL
    xs = _s3(64 * 64 * 128, 64 * 128, 128)
    args = (FAKE, xs, None, None, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 1, 64, 128, 512, 1)
    assert lib.of3_transition_fwd_ws(*args, FAKE, need - 1, L.OF3_DTYPE_F32, None) == L.OF3_ENOSPC
    assert lib.of3_transition_fwd_ws(*args, FAKE + 4, need, L.OF3_DTYPE_F32, None) == L.OF3_EINVAL  # workspace alignment
