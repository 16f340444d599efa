"""Regenerates inception_v3_dp_parallel_merge.json with the deterministic analytic cost model."""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, '..', '..', 'inter-operator-scheduler_amd'))

import ios  # noqa: E402

graph = ios.models.inception_v3()
optimized = ios.optimize(graph, 1, ios.AnalyticCostModel(launch=1.0, rate=2e7, sync=1.5), 'dp_parallel_merge')
with open(os.path.join(HERE, 'inception_v3_dp_parallel_merge.json'), 'w') as f:
    json.dump(optimized.export_config(), f)
