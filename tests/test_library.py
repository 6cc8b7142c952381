"""Where built libraries are looked for and written (no GPU)."""
import os
import stat

import pytest

from inferflux_amd.kernels import library


def test_the_fallback_folder_must_be_private_and_ours(tmp_path, monkeypatch):
    monkeypatch.setattr(library.tempfile, "gettempdir", lambda: str(tmp_path))
    d = tmp_path / f"inferflux_amd-{os.getuid()}"
    assert library._fallback_dir() is None and not d.exists()           # looking a library up creates nothing
    assert library._fallback_dir(create=True) == str(d) and stat.S_IMODE(os.lstat(d).st_mode) == 0o700
    os.chmod(d, 0o777)                                                   # others may write: whatever is in it is not trusted
    with pytest.raises(library.KernelBuildError, match="not a private folder"):
        library._fallback_dir()
    with pytest.raises(library.KernelBuildError, match="not a private folder"):
        library.find_library("ceilings", (("NO_SUCH_VARIANT", 1),))
    os.chmod(d, 0o700)
    os.rmdir(d)
    os.symlink(tmp_path, d)                                              # a link somebody planted under the expected name
    with pytest.raises(library.KernelBuildError, match="not a private folder"):
        library._fallback_dir(create=True)
