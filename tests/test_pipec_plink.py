"""The .plink container and canonical JSON: closed-form byte-level checks
(pipec/src/pipec2/container.py:14-62 and canonjson.py:8-11 fix every parameter)."""
import io
import json
import zipfile

import pytest

from pipelink_amd.pipec import plink
from pipelink_amd.pipec.clauses import PackError


def test_canonical_json_is_sorted_compact_lf_terminated():
    assert plink.canonical_dumps({"b": [1, 2.5, None, True], "a": {"z": "x", "y": 0}}) == \
        '{"a":{"y":0,"z":"x"},"b":[1,2.5,null,true]}\n'
    with pytest.raises(ValueError):
        plink.canonical_dumps({"x": float("nan")})
    assert plink.sha256_hex(b"") == "e3b0c44298fc1c149afbf4c8996fb92427ae41e4649b934ca495991b7852b855"


def test_container_layout_and_golden_digest(tmp_path):
    out = tmp_path / "a.plink"
    report = plink.pack({"payload": {"file": "stage.o"}}, b"\x00\x01\x02\x03", out)
    blob = out.read_bytes()
    # golden: computed by this implementation, cross-checked member by member below
    assert report["payload"]["sha256"] == "054edec1d0211f624fed0cbca9d4f9400b0e491c43742af2c5b0abebf0c990d8"
    assert report["manifest_sha256"] == plink.sha256_hex(
        b'{"payload":{"file":"stage.o","sha256":"054edec1d0211f624fed0cbca9d4f9400b0e491c43742af2c5b0abebf0c990d8"}}\n')
    assert report["artifact_sha256"] == plink.sha256_hex(blob)
    with zipfile.ZipFile(io.BytesIO(blob)) as zf:
        infos = zf.infolist()
        assert [i.filename for i in infos] == ["manifest.json", "stage.o"]
        for i in infos:
            assert i.date_time == (1980, 1, 1, 0, 0, 0) and i.compress_type == zipfile.ZIP_DEFLATED
            assert i.create_system == 3 and i.external_attr == 0o600 << 16 and i.extra == b"" and i.comment == b""
        assert zf.comment == b""
        assert zf.read("stage.o") == b"\x00\x01\x02\x03"
    # deterministic: packing again gives the same bytes
    plink.pack({"payload": {"file": "stage.o"}}, b"\x00\x01\x02\x03", tmp_path / "b.plink")
    assert (tmp_path / "b.plink").read_bytes() == blob
    manifest, payload = plink.read(out)
    assert payload == b"\x00\x01\x02\x03" and manifest["payload"]["sha256"] == report["payload"]["sha256"]


@pytest.mark.parametrize("manifest,where", [
    ({}, "$.payload"),
    ({"payload": {"file": "other.o"}}, "$.payload.file"),
    ({"payload": {"file": "stage.o", "sha256": "00"}}, "$.payload.sha256"),
    ({"payload": {"file": "stage.o", "size": 1}}, "$.payload.size"),
])
def test_source_manifest_rules(tmp_path, manifest, where):
    with pytest.raises(PackError) as err:
        plink.pack(manifest, b"x", tmp_path / "x.plink")
    assert err.value.clause_ids == {"P-CONTAINER"} and err.value.failures[0].path == where


def test_read_rejects_garbage_and_tampered_payload(tmp_path):
    bad = tmp_path / "bad.plink"
    bad.write_bytes(b"not a zip")
    with pytest.raises(PackError):
        plink.read(bad)
    good = tmp_path / "g.plink"
    plink.pack({"payload": {"file": "stage.o"}}, b"abcd", good)
    with zipfile.ZipFile(good) as zf:
        manifest = zf.read("manifest.json")
    tampered = tmp_path / "t.plink"
    with zipfile.ZipFile(tampered, "w") as zf:
        zf.writestr("manifest.json", manifest)
        zf.writestr("stage.o", b"abce")
    with pytest.raises(PackError) as err:
        plink.read(tampered)
    assert "digest" in str(err.value)
