"""Installs the package that lives in ``jax-llm-examples_amd/`` under its import name
``jax_llm_examples_amd``.  The HIP sources travel with it and are compiled for gfx950 on first use
(``ops/build.py``), so installing needs no GPU and no ROCm."""
from setuptools import setup

SUB = ["cache", "config", "engine", "ops", "parts", "sampling", "weights", "csrc"]

setup(
    name="jax_llm_examples_amd",
    version="0.1.0",
    description="A one-GPU inference engine for Llama 4 on AMD MI355X (gfx950): PyTorch-ROCm tensors and "
                "hand-written HIP kernels",
    python_requires=">=3.10",
    license="Apache-2.0",
    install_requires=["torch", "numpy"],
    packages=["jax_llm_examples_amd"] + [f"jax_llm_examples_amd.{s}" for s in SUB],
    package_dir={"jax_llm_examples_amd": "jax-llm-examples_amd"},
    package_data={"jax_llm_examples_amd.csrc": ["*.hip", "*.h"]},
    scripts=["bin/trace_run"],
    entry_points={"console_scripts": ["jax-llm-examples-amd = jax_llm_examples_amd.main:main"]},
)
