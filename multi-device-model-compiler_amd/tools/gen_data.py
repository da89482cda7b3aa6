#!/usr/bin/env python3
"""Seeded input files for the runners.

Same file convention as the reference's examples/data_util.py:44-59 (raw
little-endian array, named ``<out>_<dtype>_<d0_d1_...>.dat``), but every draw
comes from ``numpy.random.Generator(PCG64(seed))`` so a run can be repeated,
and the distribution can be chosen: ``random`` is the reference's U[0,1),
``uniform`` is U[-1,1), ``normal`` is N(mean, std).
"""
from __future__ import annotations

import argparse

import numpy as np

DTYPES = {"f32": np.float32, "f16": np.float16}


def parse_shape(shape: str):
    return [int(s) for s in shape.split("_")]


def print_shape(shapes) -> str:
    return "_".join(str(s) for s in shapes)


def load_data_raw(file_name: str, type: str = "f32"):
    return np.fromfile(file_name, dtype=DTYPES[type])


def load_data(file_name: str, shape: str, type: str = "f32"):
    return np.fromfile(file_name, dtype=DTYPES[type]).reshape(parse_shape(shape))


def gen_data(shape: str, type: str = "f32", seed: int = 0, dist: str = "random", mean: float = 0.0,
             std: float = 1.0):
    rng = np.random.Generator(np.random.PCG64(seed))
    shapes = parse_shape(shape)
    if dist == "random":
        data = rng.random(shapes)
    elif dist == "uniform":
        data = rng.uniform(-1.0, 1.0, shapes)
    elif dist == "normal":
        data = mean + std * rng.standard_normal(shapes)
    else:
        raise NotImplementedError("Not Implemented distribution!")
    return data.astype(DTYPES[type])


def save_data(array: np.ndarray, output_name: str) -> str:
    file_name = f"{output_name}_{array.dtype}_{print_shape(array.shape)}.dat"
    array.tofile(file_name, sep="")
    return file_name


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--shape", type=str, required=True, help="Gen data shape")
    ap.add_argument("-o", "--output", type=str, default="data", help="output name")
    ap.add_argument("--type", type=str, default="f32", help="data type")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--dist", type=str, default="random", choices=["random", "uniform", "normal"])
    ap.add_argument("--mean", type=float, default=0.0)
    ap.add_argument("--std", type=float, default=1.0)
    a = ap.parse_args()
    print(save_data(gen_data(a.shape, a.type, a.seed, a.dist, a.mean, a.std), a.output))


if __name__ == "__main__":
    main()
