"""Re-pack the reference's HMM test fixtures as .npz files.

The reference keeps its golden inputs as HDF5 (test/data/{3mer,5mer}-model.hdf5,
test/data/signals.hdf5) and reads them with h5py (test/test_forward.py:31-77).
h5py is not installed here, so this script shells out to the HDF5 command line
tools (h5dump/h5ls) and stores the *raw* tables unchanged; all layout
transformations (log, reshape, k-mer index reversal) happen in the oracle.

Outputs (committed next to this script):
  hmm_3mer_model.npz, hmm_5mer_model.npz : obs [101,4^k], trans [4,4^k],
      duration [16], tail_factor (scalar), k (scalar); dtype as stored.
  hmm_signals.npz : concatenated int16 signal samples + per-read lengths +
      read names, in HDF5 name order (the order h5py's keys() yields).
  hmm_{3,5,7}mer_expected.txt : copies of the reference's expected
      log-likelihood files (data, 100 floats each).

Usage: python tests/golden/make_fixtures.py [/root/reference]
"""
import os
import re
import shutil
import subprocess
import sys
import tempfile

import numpy as np

H5DUMP = shutil.which("h5dump") or "/opt/conda/bin/h5dump"
H5LS = shutil.which("h5ls") or "/opt/conda/bin/h5ls"
HERE = os.path.dirname(os.path.abspath(__file__))

_DT = {"H5T_IEEE_F64LE": "<f8", "H5T_IEEE_F32LE": "<f4", "H5T_STD_I16LE": "<i2",
       "H5T_STD_I64LE": "<i8", "H5T_STD_U32LE": "<u4"}


def _header(path, obj, flag="-d"):
    out = subprocess.run([H5DUMP, "-H", flag, obj, path], check=True,
                         capture_output=True, text=True).stdout
    dt = re.search(r"DATATYPE\s+(\S+)", out).group(1)
    m = re.search(r"SIMPLE \{ \(([^)]*)\)", out)
    shape = tuple(int(x) for x in m.group(1).split(",")) if m else ()
    return _DT[dt], shape


def read_dataset(path, dset):
    dt, shape = _header(path, dset)
    with tempfile.NamedTemporaryFile(suffix=".bin") as tmp:
        subprocess.run([H5DUMP, "-d", dset, "-b", "LE", "-o", tmp.name, path],
                       check=True, capture_output=True)
        return np.fromfile(tmp.name, dtype=dt).reshape(shape)


def read_attr(path, attr):
    dt, _ = _header(path, attr, "-a")
    out = subprocess.run([H5DUMP, "-m", "%.17g", "-a", attr, path], check=True,
                         capture_output=True, text=True).stdout
    val = re.search(r"\(0\):\s*(\S+)", out).group(1)
    return np.array(float(val) if "f" in dt else int(val)).astype(dt)


def pack_model(ref, k):
    src = f"{ref}/test/data/{k}mer-model.hdf5"
    np.savez_compressed(
        f"{HERE}/hmm_{k}mer_model.npz",
        obs=read_dataset(src, "/Tables/ObservationProbabilities"),
        trans=read_dataset(src, "/Tables/TransitionProbabilities"),
        duration=read_dataset(src, "/Tables/DurationProbabilities"),
        tail_factor=read_attr(src, "/Tables/DurationProbabilities/TailFactor"),
        k=read_attr(src, "/Parameters/KMerLength"))


def pack_signals(ref):
    src = f"{ref}/test/data/signals.hdf5"
    out = subprocess.run([H5LS, src], check=True, capture_output=True, text=True).stdout
    names = [l.split()[0] for l in out.splitlines() if l.strip()]
    sigs = [read_dataset(src, f"/{n}/Raw/Signal") for n in names]
    np.savez_compressed(
        f"{HERE}/hmm_signals.npz",
        samples=np.concatenate(sigs).astype(np.int16),
        lens=np.array([len(s) for s in sigs], dtype=np.int64),
        names=np.array(names))


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    for k in (3, 5):
        pack_model(ref, k)
    pack_signals(ref)
    for k in (3, 5, 7):
        shutil.copyfile(f"{ref}/test/data/{k}mer-expected.txt",
                        f"{HERE}/hmm_{k}mer_expected.txt")


if __name__ == "__main__":
    main()
