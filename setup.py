"""Packaging of flyvec_amd.  The console scripts carry the reference's names (settings.ini:19-20)."""
from setuptools import find_packages, setup

setup(
    name="flyvec_amd",
    version="0.1.0",
    description="FlyVec training step and top-k hashing on AMD MI355X (HIP, gfx950)",
    packages=find_packages(include=["flyvec_amd", "flyvec_amd.*"]),
    package_data={"flyvec_amd": ["csrc/*", "lib/*.so"]},
    python_requires=">=3.8",
    install_requires=["numpy"],
    entry_points={"console_scripts": ["flyvec_train=flyvec_amd.train_flyvec:main",
                                      "flyvec_compile=flyvec_amd.train_flyvec:init"]},
)
