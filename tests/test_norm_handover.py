"""The norm that rides on the products around it, on the CPU: which of its three forms a step takes (half done with a
row factor for the product behind it; finished by the product before it; a kernel of its own) is decided by the
parts among themselves from what the kernel set says it can do. A stand-in kernel set with small limits walks a
tiny model through all three, and the logits must not depend on the form."""
import pytest
import torch

from helpers import TOL, make_folder, random_tokens, read_folder, rel_err
from kernel_double import KernelDouble
from reinfer_amd import kernels
from reinfer_amd.engine import ModelRunner, StepEntry


class HandOver(KernelDouble):
    """Up to 4 rows the half-done form, 5 to 12 rows the finished form for products with an even K / 16, else none."""
    NORM_ON_PRODUCTS_ROWS = 4
    NORM_FINISHED_ROWS = 12

    def __init__(self):
        self.emitted = self.finished = self.declined = 0

    def can_accumulate(self, x, weight):
        return True

    def can_finish_norm(self, M, N, K):
        return self.NORM_ON_PRODUCTS_ROWS < M <= self.NORM_FINISHED_ROWS and (K // 16) % 2 == 0

    def linear_skinny(self, x, weight, out, bias=None, accumulate=False, row_sums=None, emit=None, finish=None):
        if finish is None:
            if emit is not None:
                self.emitted += 1
            return super().linear_skinny(x, weight, out, bias, accumulate, row_sums, emit)
        assert accumulate and row_sums is None and emit is None
        super().linear_skinny(x, weight, out, bias, True)
        if not self.can_finish_norm(x.shape[0], weight.shape[0], x.shape[1]):
            self.declined += 1
            return False
        w, xo, eps = finish
        y = out.float()
        xo.copy_((y * torch.rsqrt((y * y).mean(dim=1, keepdim=True) + eps) * w.float()).to(xo.dtype))
        self.finished += 1
        return True


class NoHandOver(KernelDouble):
    skinny_row_parts = None
    NORM_ON_PRODUCTS_ROWS = 0


@pytest.mark.parametrize("which", ["A", "B"])
def test_the_three_forms_of_a_norm_give_the_same_logits(tmp_path, which):
    folder = make_folder(tmp_path, which, "bfloat16")
    raw, _ = read_folder(folder)
    for T, form in ((3, "emitted"), (9, "finished"), (20, None)):
        toks = random_tokens(T, raw["vocab_size"], 31 + T)
        got = {}
        for name, ops in (("with", HandOver()), ("without", NoHandOver())):
            with kernels.use(ops):
                runner = ModelRunner.from_folder(folder, dtype="bfloat16", device="cpu", max_tokens=64)
                runner.add_request("a")
                got[name] = runner.step([StepEntry("a", toks, list(range(T)))])
            if name == "with":
                counts = {"emitted": ops.emitted, "finished": ops.finished + ops.declined}
                for k, v in counts.items():
                    assert (v > 0) == (k == form), (T, counts)
                if form == "finished":
                    # tiny B's feed-forward width is no even number of 16s: its down projection declines, and
                    # the norm behind it runs as a kernel; every other product finishes its norm
                    assert ops.finished > 0 and (ops.declined > 0) == ((raw["intermediate_size"] // 16) % 2 == 1
                                                                       or (raw["num_attention_heads"] * raw["head_dim"] // 16) % 2 == 1)
        assert torch.isfinite(got["with"]).all()
        if form == "emitted":
            # the half-done form rounds stream * weight to bfloat16 before the product instead of the normed row
            # behind it: one rounding of 2^-9 a norm in another place (measured 2e-3 to 5e-3)
            assert rel_err(got["with"], got["without"]) < TOL["bfloat16"], (T, form)
        else:
            # the finished form is the norm kernel's arithmetic in another kernel: the same bits in this stand-in
            assert torch.equal(got["with"], got["without"]), (T, form)
