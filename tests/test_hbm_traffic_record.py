"""The counter-traffic record behind bench.py's `roofline.traffic` (host logic, no GPU): entries
are made from rocprofv3 counter CSVs, scaled by the calibration copy, keyed by workload and
variant, and valid only for the kernel sources they were measured on."""
import csv
import json
import os

import pytest

from quantfour_adamw_cuda_amd import hbm_traffic as ht

FIELDS = ["Kernel_Name", "Counter_Name", "Counter_Value", "Grid_Size"]
COPY = "void q4::probe_move_kernel<0>(q4::ProbeArgs)"
STEP = "void q4::fused_4bit_kernel<0, 1, false, false>(q4::FusedArgs)"
SMALL = "void q4::single_tensor_kernel<0, 1, false>(q4::SmallArgs)"


def _write(path, counter, rows):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=FIELDS)
        w.writeheader()
        for name, value in rows:
            w.writerow({"Kernel_Name": name, "Counter_Name": counter, "Counter_Value": value, "Grid_Size": 256})


def test_record_scales_by_the_copy_and_lookup_follows_the_sources(tmp_path, monkeypatch):
    # the fetch counter reports half of the KiB read (as on the MI355X), the write counter all of them
    four_gib_kib = float(4 << 20)
    fetch = str(tmp_path / "f" / "node" / "1_counter_collection.csv")
    write = str(tmp_path / "w" / "node" / "1_counter_collection.csv")
    steps = 4
    _write(fetch, "FETCH_SIZE", [(COPY, four_gib_kib / 2)] * 3 + [(STEP, 1000.0), (STEP, 3000.0), (SMALL, 10.0)] * steps
           + [("at::native::some_torch_kernel", 1e9)])
    _write(write, "WRITE_SIZE", [(COPY, four_gib_kib)] * 3 + [(STEP, 1500.0), (STEP, 4500.0), (SMALL, 20.0)] * steps)
    out = str(tmp_path / "record.json")
    e = ht.record("llama3-8b", "group", "real-nearest", [str(tmp_path / "f" / "**" / "*counter_collection.csv")],
                  [str(tmp_path / "w" / "**" / "*counter_collection.csv")], steps, out, profile="profiles/x.txt")
    assert e["fetch_scale"] == pytest.approx(2.0) and e["write_scale"] == pytest.approx(1.0)
    assert e["fetch_bytes_per_step"] == pytest.approx((1000 + 3000 + 10) * 1024 * 2.0)
    assert e["write_bytes_per_step"] == pytest.approx((1500 + 4500 + 20) * 1024)
    assert e["bytes_per_step"] == e["fetch_bytes_per_step"] + e["write_bytes_per_step"]
    assert e["dispatches_per_step"] == 3 and e["kernels"] == sorted([STEP, SMALL])
    # a second variant lands beside the first
    ht.record("llama3-8b", "rank1", "real-nearest", [fetch], [write], steps, out)
    doc = json.load(open(out))
    assert set(doc["entries"]) == {"llama3-8b|group|real-nearest", "llama3-8b|rank1|real-nearest"}
    assert ht.lookup("llama3-8b", path=out)["bytes_per_step"] == e["bytes_per_step"]
    assert ht.lookup("llama2-13b", path=out) is None                       # never recorded
    assert ht.lookup("llama3-8b", path=str(tmp_path / "missing.json")) is None
    # the kernels change: the number is no longer theirs
    monkeypatch.setattr(ht, "source_hash", lambda: "0" * 16)
    assert ht.lookup("llama3-8b", path=out) is None


def test_written_bytes_from_an_earlier_record_carry_their_provenance(tmp_path, monkeypatch):
    """a WRITE_SIZE session that could not be taken on the present sources: the entry takes that
    half from an earlier record, names the sources it was measured on and says why it still holds"""
    four_gib_kib = float(4 << 20)
    fetch = str(tmp_path / "f.csv")
    write = str(tmp_path / "w.csv")
    _write(fetch, "FETCH_SIZE", [(COPY, four_gib_kib / 2)] + [(STEP, 1000.0), (SMALL, 10.0)] * 2)
    _write(write, "WRITE_SIZE", [(COPY, four_gib_kib)] + [(STEP, 1500.0), (SMALL, 20.0)] * 2)
    earlier = str(tmp_path / "earlier.json")
    monkeypatch.setattr(ht, "source_hash", lambda: "a" * 16)
    e0 = ht.record("llama3-8b", "group", "real-nearest", [fetch], [write], 2, earlier)
    monkeypatch.setattr(ht, "source_hash", lambda: "b" * 16)
    out = str(tmp_path / "record.json")
    with pytest.raises(SystemExit, match="write-note"):
        ht.record("llama3-8b", "group", "real-nearest", [fetch], [], 2, out, write_from_record=earlier)
    with pytest.raises(SystemExit, match="no entry"):
        ht.record("gpt2-small", "group", "real-nearest", [fetch], [], 2, out, write_from_record=earlier, write_note="x")
    e = ht.record("llama3-8b", "group", "real-nearest", [fetch], [], 2, out, write_from_record=earlier,
                  write_note="same instructions")
    assert e["source_hash"] == "b" * 16 and e["write_source_hash"] == "a" * 16 and e["write_note"] == "same instructions"
    assert e["fetch_bytes_per_step"] == pytest.approx(e0["fetch_bytes_per_step"])
    assert e["write_bytes_per_step"] == e0["write_bytes_per_step"]
    assert e["bytes_per_step"] == pytest.approx(e["fetch_bytes_per_step"] + e["write_bytes_per_step"])
    assert ht.lookup("llama3-8b", path=out)["write_source_hash"] == "a" * 16     # valid for the present sources
    import bench
    assert "a" * 16 in bench.traffic_source(e) and "same instructions" in bench.traffic_source(e)
    assert "WRITE_SIZE" not in bench.traffic_source(e0)
    # the sources change once more and no session can be taken: the entry is carried over whole,
    # keeps the sources of both of its sessions and gains the reason
    monkeypatch.setattr(ht, "source_hash", lambda: "c" * 16)
    assert ht.lookup("llama3-8b", path=out) is None
    carried = str(tmp_path / "carried.json")
    with pytest.raises(SystemExit, match="note"):
        ht.restamp(out, carried, None)
    with pytest.raises(SystemExit, match="no entry"):
        ht.restamp(out, carried, "why", keys=["gpt2-small|group|real-nearest"])
    (c,) = ht.restamp(out, carried, "one wait state more")
    assert (c["source_hash"], c["fetch_source_hash"], c["write_source_hash"]) == ("c" * 16, "b" * 16, "a" * 16)
    assert c["bytes_per_step"] == e["bytes_per_step"] and ht.lookup("llama3-8b", path=carried)["note"] == "one wait state more"
    text = bench.traffic_source(c)
    assert "FETCH_SIZE session ran on sources " + "b" * 16 in text and "WRITE_SIZE session ran on sources " + "a" * 16 in text
    assert "one wait state more" in text and "same instructions" in text


def test_a_profile_without_the_calibration_copy_is_refused(tmp_path):
    fetch = str(tmp_path / "f.csv")
    write = str(tmp_path / "w.csv")
    _write(fetch, "FETCH_SIZE", [(STEP, 1000.0)])
    _write(write, "WRITE_SIZE", [(COPY, 4194304.0), (STEP, 1000.0)])
    with pytest.raises(SystemExit, match="calibrate-copy"):
        ht.record("llama3-8b", "group", "real-nearest", [fetch], [write], 1, str(tmp_path / "r.json"))


def test_source_hash_covers_the_kernel_sources_only(tmp_path, monkeypatch):
    """the hash follows csrc/q4adamw*.hip and csrc/q4adamw_*.h, and nothing else in the folder"""
    h0 = ht.source_hash()
    assert len(h0) == 16 and h0 == ht.source_hash()
    csrc = tmp_path / "pkg" / "csrc"
    csrc.mkdir(parents=True)
    (csrc / "q4adamw.hip").write_text("a")
    (csrc / "q4adamw_step.h").write_text("b")
    (csrc / "q4stream_probe.hip").write_text("c")
    monkeypatch.setattr(ht, "_HERE", str(tmp_path / "pkg"))
    h1 = ht.source_hash()
    (csrc / "q4stream_probe.hip").write_text("changed")
    (csrc / "libq4adamw.so").write_text("binary")
    assert ht.source_hash() == h1
    (csrc / "q4adamw_step.h").write_text("changed")
    h2 = ht.source_hash()
    assert h2 != h1
    (csrc / "q4adamw_pick_fused.hip").write_text("a kernel's instantiations")
    assert ht.source_hash() != h2


def test_committed_record_is_well_formed():
    with open(ht.DEFAULT_PATH) as f:
        doc = json.load(f)
    assert doc["entries"], "profiles/hbm_traffic.json holds no entry"
    for key, e in doc["entries"].items():
        workload, variance, rounding, *form = key.split("|")
        assert variance in ("group", "rank1") and rounding in ("real-nearest", "stochastic")
        assert form in ([], ["exact"], ["folded"])
        assert e["bytes_per_step"] == pytest.approx(e["fetch_bytes_per_step"] + e["write_bytes_per_step"])
        assert 1.9 < e["fetch_scale"] < 2.1 and 0.95 < e["write_scale"] < 1.05
        assert len(e["source_hash"]) == 16 and e["dispatches_per_step"] >= 1
        for half in ("fetch", "write"):   # a half measured on other sources says which, and the entry why
            h = e.get(half + "_source_hash", e["source_hash"])
            assert len(h) == 16
            if h != e["source_hash"]:
                assert len(e.get("note", "")) > 20 or len(e.get("write_note", "")) > 20
