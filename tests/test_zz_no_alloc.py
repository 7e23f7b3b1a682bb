"""The allocation-free entry point mi_launch_packed_scratch against mi_launch_packed.

The per-column mean / variance / argmax pair keeps its per-split partials in a workspace: through
mi_launch_packed the caller brings a torch allocation, through mi_launch_packed_scratch the library
substitutes its fixed per-GPU array.  Same kernels, same launch shapes, so the outputs must be
bit-identical (fp32 words and int64 indices compared as integers).  Two calls in a row share the
array, the second on a smaller input, so stale partials of the first call lie beyond what the second
one writes.  Collected last (file name) so a failure here hides no other test.
"""
import ctypes

import numpy as np
import pytest
import torch

from tests.helpers import announce

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    a, b = a.cpu().contiguous(), b.cpu().contiguous()
    if a.dtype == torch.float32:
        a, b = a.view(torch.int32), b.view(torch.int32)
    return bool(torch.equal(a, b))


def test_scratch_launch_matches_workspace_launch_twice_in_a_row():
    from inductor_x_amd import kernels as K
    from inductor_x_amd import launcher

    lib = launcher.load_library()
    cap = ctypes.c_size_t(0)
    assert lib.mi_scratch_capacity(ctypes.byref(cap)) == 0 and cap.value == 8 << 20
    torch.manual_seed(11)
    for rows, cols in [(65536, 512), (3001, 256)]:  # second call: smaller input, fewer partials
        announce(f"library-scratch col stats rows={rows} cols={cols}")
        x = torch.randn(rows, cols, device=DEV)
        x[rows // 3, 5] = x[rows // 2, 5] = 9.0  # a tie across splits
        ref = K.col_mean_var_argmax(x)
        out = (
            torch.full((cols,), float("nan"), device=DEV),
            torch.full((cols,), float("nan"), device=DEV),
            torch.full((cols,), -1, dtype=torch.int64, device=DEV),
        )
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
        got = K.col_mean_var_argmax(x, workspace="library", out=out)
        after = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
        torch.cuda.synchronize()
        assert after == before, "the library-scratch call allocated through torch"
        for g, r, name in zip(got, ref, ("mean", "var", "argmax")):
            assert _same_bits(g, r), f"{name} differs between the scratch and the workspace launch"
        assert np.array_equal(got[2].cpu().numpy(), torch.argmax(x, 0).cpu().numpy())


def test_scratch_request_beyond_capacity_is_refused():
    from inductor_x_amd import kernels as K
    from inductor_x_amd import launcher

    announce("library-scratch over capacity")
    x = torch.randn(4096, 64, device=DEV)
    K.col_mean_var_argmax(x)  # loads the kernels
    lp = K._col_partial_launcher()
    fn = lp.launchers[0][1]
    with pytest.raises(launcher.LauncherError, match="scratch"):
        fn.launch_with_library_scratch("PPiii", (x.data_ptr(), 0, 4096, 64, 1), 1, (8 << 20) + 1, (1, 1, 1), (256,), 0)
    torch.cuda.synchronize()
