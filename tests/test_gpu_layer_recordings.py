"""The two recordings of a whole layer between its projections that `bench.py --layer` times (the reference's seven
operators, crates/inference-executor-metal/src/attn/gqa/backend.rs:358-421, and this library's three launches) leave the
same output and page bytes, replayed from a HIP graph, on the decode batch of config 2 with both page formats and on the
chunked-prefill batch of config 5, whose Map writes the output itself."""
import pytest

import bench

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("index,fp8_pages", [(2, False), (2, True), (5, False)])
def test_shortest_recording_leaves_the_bytes_of_the_seven_operators(device, index, fp8_pages):
    print(f"layer recordings of config {index} fp8_pages={fp8_pages}", flush=True)
    row = bench.layer_rows(device, index, fp8_pages=fp8_pages, replays=3)
    assert row["same_output_bytes"] and row["same_page_bytes"]
    assert row["launches_shortest_recording"] == (2 if index == 5 else 3)
    assert 0 < row["shortest_recording_us"] and 0 < row["reference_recording_us"]
