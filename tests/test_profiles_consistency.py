"""bench.py's `roofline.traffic` constants are the HBM bytes of the committed counter summaries under profiles/."""
import os
import re

import bench

PROFILES = {2: ("split_kv_map_kernel_config2_decode.txt", "split_kv_map_kernel"),
            3: ("split_kv_map_kernel_config3_long_context_gated.txt", "split_kv_map_kernel"),
            4: ("tile_map_kernel_config4_spec_verify.txt", "tile_map_kernel"),
            5: ("tile_map_kernel_config5_chunked_prefill.txt", "tile_map_kernel"),
            6: ("tile_map_kernel_extra_prefill_d256.txt", "tile_map_kernel")}


def test_measured_traffic_constants_match_the_committed_profiles():
    cases = [(index, name, kernel, bench.MEASURED_MAP_TRAFFIC_BYTES) for index, (name, kernel) in PROFILES.items()]
    cases += [(index, name.replace(".txt", "_fp8_pages.txt"), kernel, bench.MEASURED_MAP_TRAFFIC_BYTES_FP8_PAGES)
              for index, (name, kernel) in PROFILES.items()]
    for index, name, kernel, constants in cases:
        text = open(os.path.join(bench.ROOT, "profiles", name)).read()
        factors = re.search(r"scale factors ([\d.]+) \(FETCH_SIZE\) and ([\d.]+) \(WRITE_SIZE\)", text)
        assert factors, name
        fetch_factor, write_factor = float(factors.group(1)), float(factors.group(2))
        row = re.search(r"khm::" + kernel + r"<[^>]*>\s+FETCH_SIZE\s+(\d+) ->.*WRITE_SIZE\s+(\d+) ->", text)
        assert row, name
        measured = (int(row.group(1)) * fetch_factor + int(row.group(2)) * write_factor) * 1024
        # the scale factors are printed with three decimals
        assert abs(measured - constants[index]) <= 1e-3 * measured, (name, measured)
