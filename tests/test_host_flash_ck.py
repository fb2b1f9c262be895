"""CPU-only: the package and module names of the reference resolve (`flash_ck`, `flash_ck.ops.fmha`, `flash_ck.nn`,
the compiled `flash_ck.flash_ck`), the FMHA family is registered, and the compiled functions validate their tensors
before anything reaches the C ABI."""
import pytest
import torch

flash_ck = pytest.importorskip("flash_ck", reason="python -m flash_ck.build has not been run")

OPS = ["fmha_fwd", "fmha_fwd_varlen", "fmha_fwd_splitkv", "fmha_fwd_splitkv_combine", "fmha_fwd_appendkv", "fmha_batch_prefill",
       "fmha_fwd_pagedkv"]


def test_names_of_the_reference_resolve():
    import flash_ck.flash_ck as compiled            # TORCH_EXTENSION_NAME of core/pybind/pybind.cc:13
    for name in OPS + ["fmha_num_splits_heuristic", "fmha_version"]:
        assert callable(getattr(compiled, name)) and getattr(flash_ck, name) is getattr(compiled, name)
    for name in OPS:
        assert callable(getattr(flash_ck.ops.fmha, name)), name
    assert flash_ck.nn.Attention is flash_ck.Attention
    assert flash_ck.is_available("fmha") and flash_ck.get_available_operations()["fmha"] is True
    from flash_ck.utils import FlashCKOperationType, get_flashck_functions
    assert get_flashck_functions(FlashCKOperationType.FMHA.value)["forward"] is flash_ck.ops.fmha.fmha_fwd
    assert flash_ck.get_flag_value("FC_TUNING_SEED") == "42"
    with pytest.raises(RuntimeError, match="Flag not found"):
        flash_ck.get_flag_value("FC_NO_SUCH_FLAG")


def test_heuristic_matches_the_c_abi():
    from flashck_amd.ops import fmha
    for args in [(4, 64, 8, 1, 32768, 128, 256), (32, 32, 8, 1, 4096, 128, 256), (1, 8, 8, 1, 100, 64, 256)]:
        assert flash_ck.fmha_num_splits_heuristic(*args) == fmha.num_splits_heuristic(*args)


def test_compiled_functions_validate_their_tensors():
    h = torch.zeros(1, 4, 2, 64, dtype=torch.float16)
    i32 = torch.zeros(2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="q must be a GPU tensor"):
        flash_ck.fmha_fwd(h, h, h)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        flash_ck.fmha_fwd_splitkv(h, h, h, 2, i32, torch.zeros(1, 1, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        flash_ck.fmha_fwd_splitkv_combine(torch.zeros(1, 2, 2, 1), torch.zeros(1, 2, 2, 1, 64), torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        flash_ck.fmha_fwd_appendkv(None, h, h, h, h, i32, torch.zeros(1, 1, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        flash_ck.fmha_batch_prefill(h[0], h, h, i32, i32, i32, max_seqlen_q=4)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        flash_ck.fmha_fwd_pagedkv(h, h, h, i32, torch.zeros(1, 1, dtype=torch.int32))
    with pytest.raises(TypeError):
        flash_ck.fmha_fwd(h, h)                                      # arity is checked by the binding
