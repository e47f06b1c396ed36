"""Reading checkpoint files (no GPU): the loader executes nothing from the file and accepts both of torch's
serialization formats, as the reference's plain torch.load does (rwkv_pip_package/src/rwkv/model.py:641)."""
import torch

from chatrwkv_amd.model import _load_checkpoint


def test_zip_and_legacy_serialization(tmp_path):
    d = {"emb.weight": torch.randn(5, 4), "blocks.0.ln0.weight": torch.ones(4)}
    new, old = str(tmp_path / "new.pth"), str(tmp_path / "old.pth")
    torch.save(d, new)
    torch.save(d, old, _use_new_zipfile_serialization=False)     # cannot be memory-mapped
    for path in (new, old):
        w = _load_checkpoint(path)
        assert set(w) == set(d)
        for k in d:
            assert torch.equal(w[k], d[k])


def test_a_file_that_needs_code_execution_is_refused(tmp_path):
    class Evil:
        def __reduce__(self):
            return (print, ("executed",))
    path = str(tmp_path / "evil.pth")
    torch.save({"x": Evil()}, path)
    try:
        _load_checkpoint(path)
    except Exception as e:                                       # torch's UnpicklingError
        assert "weights_only" in str(e) or "Unsupported" in str(e) or "allowed" in str(e)
    else:
        raise AssertionError("a pickle that calls a function was loaded")
