"""The reference's import paths (Swin3D/modules/swin3d_layers.py:16-24) resolve to the swin3d_amd operators,
and the rest of a `Swin3D` package further down sys.path stays importable."""
import importlib
import os
import sys
import textwrap


def test_reference_import_paths_resolve_to_swin3d_amd():
    import swin3d_amd
    from Swin3D.sparse_dl.attn.attn_coff import IndexMode, PosEmb, PrecisionMode, SelfAttnAIOFunction, TableDims
    import Swin3D.sparse_dl.knn
    from Swin3D.sparse_dl.knn import KNN
    assert SelfAttnAIOFunction is swin3d_amd.SelfAttnAIOFunction
    assert KNN is swin3d_amd.sparse_dl.knn.KNN and Swin3D.sparse_dl.knn.KNN is KNN
    assert (PosEmb.SEPARATE.value, TableDims.D0.value, IndexMode.INDIRECT.value) == (3, 3, 2)
    assert [m.name for m in PrecisionMode] == ["HALF_ALL", "HALF_FORWARD", "HALF_NONE"]


def test_other_subpackages_of_a_swin3d_checkout_stay_importable(tmp_path):
    """A stand-in for the reference's checkout (a `Swin3D` package with a `modules` sub-package that imports its
    operators the reference's way) placed after this repository on sys.path."""
    pkg = tmp_path / "Swin3D"
    (pkg / "modules").mkdir(parents=True)
    (pkg / "__init__.py").write_text("")
    (pkg / "modules" / "__init__.py").write_text("")
    (pkg / "modules" / "layers_standin.py").write_text(textwrap.dedent("""
        from Swin3D.sparse_dl.attn.attn_coff import SelfAttnAIOFunction, PosEmb, TableDims, IndexMode, PrecisionMode
        import Swin3D.sparse_dl.knn
        from Swin3D.sparse_dl.knn import KNN
    """))
    sys.path.append(str(tmp_path))
    saved = {k: sys.modules.pop(k) for k in list(sys.modules) if k == "Swin3D" or k.startswith("Swin3D.")}
    try:
        mod = importlib.import_module("Swin3D.modules.layers_standin")
        import swin3d_amd
        assert mod.SelfAttnAIOFunction is swin3d_amd.SelfAttnAIOFunction
        assert os.path.dirname(mod.__file__) == str(pkg / "modules")
    finally:
        sys.path.remove(str(tmp_path))
        for k in [k for k in sys.modules if k == "Swin3D" or k.startswith("Swin3D.")]:
            del sys.modules[k]
        sys.modules.update(saved)
