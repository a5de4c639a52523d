"""Writes kmeans_sklearn.json: inertia of scikit-learn's KMeans (k-means++ initialisation, one start, 300 iterations)
on small seeded samples, the yardstick for the k-means that stands in for cuvs::cluster::kmeans::fit (third party,
not in the reference tree; call site partition.cuh:48-54).  Run from the repository root:

    python tests/golden/make_kmeans_golden.py

scikit-learn is only needed here; the tests read the JSON."""
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
from glide_amd import datasets as D      # noqa: E402

CASES = [
    # name, generator arguments, clusters
    ("mixture16-dim32-k16", dict(num=4000, dim=32, components=16, seed=5, mixture_seed=3), 16),
    ("mixture64-dim128-k16", dict(num=5000, dim=128, components=64, seed=1234, mixture_seed=99), 16),
    ("mixture16-dim32-k8", dict(num=4000, dim=32, components=16, seed=5, mixture_seed=3), 8),
]


def main():
    import sklearn
    from sklearn.cluster import KMeans
    out = {"scikit_learn": sklearn.__version__, "cases": []}
    for name, gen, k in CASES:
        x = D.gmm_clipped(**gen)
        inertias = [float(KMeans(n_clusters=k, init="k-means++", n_init=1, max_iter=300, tol=1e-4, random_state=r).fit(x).inertia_)
                    for r in range(8)]
        out["cases"].append(dict(name=name, generator="glide_amd.datasets.gmm_clipped", arguments=gen, clusters=k, random_states=list(range(8)),
                                 inertia=inertias, median=float(np.median(inertias))))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kmeans_sklearn.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print(path)


if __name__ == "__main__":
    main()
