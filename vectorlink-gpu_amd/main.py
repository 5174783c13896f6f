"""Command line driver: build an index over random unit vectors, measure its
self-recall, print and store the run as JSON under ./log/.

    python vectorlink-gpu_amd/main.py -c 100000 -d 768 -n 32 -P

Takes the flags of the reference's main.py (main.py:24-99, same letters and
defaults; note that -r and -p default to 6 and 3 there, not to the class
defaults 3 and 4).
"""
import argparse
import itertools
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

# (short flag, long flag, default, help) for the integer options; -P/--prune is the one switch
INT_OPTIONS = [
    ("-c", "--vector-count", 10_000, "number of vectors"),
    ("-d", "--vector-dimension", 1536, "dimension of vectors"),
    ("-n", "--beam_size", 24, "beam size (max number of neighbors)"),
    ("-l", "--optimization_loops", 3, "cagra loops"),
    ("-x", "--exclude_factor", 5, "factor larger than visit queue for exclusion buffer"),
    ("-q", "--visit_queue_factor", 3, "factor larger than beam for visit queue"),
    ("-f", "--beam_queue_factor", 3, "factor larger than beam for initial beams"),
    ("-b", "--batch_size", 10_000, "how many vectors/beams to run per batch"),
    ("-r", "--recall_search_queue_factor", 6, "recall search queue factor"),
    ("-p", "--parallel_visit_count", 3, "parallel visit count"),
    ("-s", "--speculative_readahead", 5, "how far to try to read-ahead before checking for progress"),
]


def parse(argv=None) -> dict:
    parser = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    for short, long_, default, text in INT_OPTIONS:
        parser.add_argument(short, long_, type=int, default=default, help=text)
    parser.add_argument("-P", "--prune", action="store_true", default=False, help="prune beams")
    return vars(parser.parse_args(argv))


def main(vectors, configuration: dict) -> dict:
    """Build, measure, and return the configuration extended with the results (reference main.py:11-21)."""
    from vectorlink_gpu.ann import ANN

    build_args = {k: v for k, v in configuration.items() if k not in ("vector_count", "vector_dimension")}
    ann = ANN(vectors=vectors, **build_args)
    report = dict(configuration)
    report.update({k: v for k, v in ann.dump_logs().items() if k in ("total_time", "recall", "gpu_arch")})
    return report


def grid_search(vector_count: int = 1_000_000, vector_dimension: int = 1536, log_dir: str = "./grid-log") -> int:
    """The reference's parameter sweep (ann.py:323-353): one build per combination, one JSON log each.
    Returns the number of experiments run."""
    from vectorlink_gpu.constants import DEVICE
    from vectorlink_gpu.utils import generate_random_vectors

    # the reference switches torch's process-wide default device here (ann.py:373-375); every tensor of
    # this package names its device instead, so the caller's default stays as it was
    fixed = {"type": "cagra", "vector_count": vector_count, "vector_dimension": vector_dimension, "exclude_factor": 5,
             "batch_size": 10_000, "beam_queue_factor": 3, "recall_search_queue_factor": 6}
    swept = {"prune": [True, False], "beam_size": [24, 32, 46], "parallel_visit_count": [1, 4],
             "optimization_loops": [1, 2], "visit_queue_factor": [3, 4]}
    vectors = generate_random_vectors(number_of_vectors=vector_count, dimensions=vector_dimension, device=DEVICE)
    os.makedirs(log_dir, exist_ok=True)
    runs = 0
    for combo in itertools.product(*swept.values()):
        configuration = dict(fixed, **dict(zip(swept.keys(), combo)))
        configuration.pop("type")
        outcome = main(vectors, configuration)
        with open(os.path.join(log_dir, f"experiment-{time.time()}.log"), "w") as sink:
            json.dump(outcome, sink)
        runs += 1
    return runs


if __name__ == "__main__":
    options = parse()
    from vectorlink_gpu.utils import generate_random_vectors

    data = generate_random_vectors(number_of_vectors=options["vector_count"], dimensions=options["vector_dimension"])
    outcome = main(data, options)
    print(outcome)
    os.makedirs("log", exist_ok=True)
    with open(os.path.join("log", f"experiment-{time.time()}.log"), "w") as sink:
        json.dump(outcome, sink)
