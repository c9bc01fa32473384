"""bench.py's table of measured memory traffic must not outlive the kernels it was measured on."""
import os

import bench


def test_measured_traffic_is_stamped_with_the_sources_it_was_measured_on():
    """Every record either carries the hash of its kernel's source files as they are now, or an
    empty one: "not measured since the kernel changed", for which bench.py reports traffic: null.
    A record whose hash names older sources fails here: measure again (the record's profile says
    how) or blank the hash."""
    for key, rec in bench.MEASURED_TRAFFIC.items():
        for f in rec["sources"] + (rec["profile"],):
            assert os.path.exists(os.path.join(bench.ROOT, f)), (key, f)
        assert rec["sha16"] in ("", bench.source_hash(rec["sources"])), \
            f"{key}: the kernel's sources changed after its traffic was measured"


def test_a_stale_record_reports_no_traffic(monkeypatch):
    key = ("gcn_powerlaw", "merge")
    rec = dict(bench.MEASURED_TRAFFIC[key], sha16="0" * 16)
    monkeypatch.setitem(bench.MEASURED_TRAFFIC, key, rec)
    traffic, provenance = bench.measured_traffic(*key, True)
    assert traffic is None and "stale" in provenance
    fresh = dict(rec, sha16=bench.source_hash(rec["sources"]))
    monkeypatch.setitem(bench.MEASURED_TRAFFIC, key, fresh)
    traffic, provenance = bench.measured_traffic(*key, True)
    assert traffic == rec["bytes"] and provenance["sha16"] == fresh["sha16"]
    assert bench.measured_traffic(*key, False) == (None, None)            # another size: not the measured launch
