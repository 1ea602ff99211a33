"""The fields of a statistics log line, searched for one by one the way the consumer of such lines does
(train_logs/process_example_logs.py:38-72 of the reference).  Test helper: the library only writes these lines."""
import re


def parse(line):
    """-> dict of the fields; ValueError when a field the consumer needs is missing"""
    found = {
        "tensor": re.search(r'Tensor\s+([\w\.]+)\s+at\s+counter\s+(\d+)\s+step\s+(\d+)', line),
        "dimension": re.search(r'tensor dimension:\s+([\dx]+)', line),
        "non_zero": re.search(r'global_non_zero:\s+(\d+)', line),
        "global_error": re.search(r'global_error:\s+([\d\.]+)', line),
        "relative_error": re.search(r'relative_error:\s+([\d\.]+)', line),
        "histogram": re.search(r'histogram\s+\[([\d,\s]+)\]', line),
    }
    missing = [k for k, m in found.items() if m is None and k != "dimension"]
    if missing:
        raise ValueError(f"not a tensor statistics line (no {', '.join(missing)}): {line!r}")
    t = found["tensor"]
    return {
        "node_id": int(line.split(':')[0].strip()),
        "tensor_name": t.group(1), "counter": int(t.group(2)), "step": int(t.group(3)),
        "tensor_dimension": found["dimension"].group(1) if found["dimension"] else None,
        "global_non_zero": int(found["non_zero"].group(1)),
        "global_error": float(found["global_error"].group(1)),
        "relative_error": float(found["relative_error"].group(1)),
        "histogram": [int(x) for x in found["histogram"].group(1).split(',')],
    }
