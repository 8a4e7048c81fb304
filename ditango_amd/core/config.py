"""Configuration object with the attribute names the hot path reads
(reference core/config.py:8-133): ``use_ditango``, ``rank``, ``local_rank``,
``num_inference_steps``, ``num_layers``, ``stride_dividers``,
``stride_percentiles``, ``model_name``, ``ditango_base``, ``use_pab`` ...
YAML keys use dashes and become underscores (config.py:66-76); WORLD_SIZE / RANK
/ LOCAL_RANK come from the environment (config.py:88-92).  The output directory
is named like the reference's (tag + timestamp) but only created on demand."""
import copy
import os
import time
from pathlib import Path

import yaml

_DEFAULTS = {
    "model_name": "cogvideox1.5-5b",
    "ditango_base": "./ditango",
    "output_fn": "./result",
    "tag": "test",
    "num_layers": 42,
    "num_inference_steps": 5,
    "seed": 42,
    "enable_timing": False,
    "do_preprocess": False,
    "do_cfg_parallel": False,
    "use_ditango": True,
    "use_ulysses": False,
    "use_distrifusion": False,
    "use_pab": False,
    "stride_dividers": [8, 4, 2, 1],
    "stride_percentiles": [20, 50, 80],
}


class DiTangoConfig:
    def __init__(self, config_path=None, **overrides):
        self.config = copy.deepcopy(_DEFAULTS)
        if config_path is not None:
            self.load_from_file(config_path)
        for k, v in overrides.items():
            self.config[k.replace("-", "_")] = v
        if self.config["do_preprocess"]:  # config.py:52-56
            for k in ("use_ditango", "use_ulysses", "use_distrifusion", "use_pab"):
                self.config[k] = False
        if not self.config["use_ditango"]:  # config.py:58-59
            self.config["stride_dividers"] = [1]
        stamp = time.strftime("%Y%m%d_%H%M")
        self.config["output_dir"] = os.path.join(self.config["output_fn"], f"{self.config['tag']}_{stamp}")
        self.config["world_size"] = int(os.getenv("WORLD_SIZE", "1"))
        self.config["rank"] = int(os.getenv("RANK", "0"))
        self.config["local_rank"] = int(os.getenv("LOCAL_RANK", "0"))

    def load_from_file(self, config_path):
        path = Path(config_path)
        if not path.exists():
            print(f"Warning: Config file {path} for DiTango not found. Using default values.")
            return
        with open(path, "r") as f:
            data = yaml.safe_load(f) or {}
        for key, value in data.items():
            self.config[key.replace("-", "_")] = value

    def __getattr__(self, name):
        cfg = self.__dict__.get("config")
        if cfg is not None and name in cfg:
            return cfg[name]
        raise AttributeError(f"'DiTangoConfig' object has no attribute '{name}'")

    def __setattr__(self, name, value):
        if name == "config":
            super().__setattr__(name, value)
        else:
            self.config[name] = value

    def to_dict(self):
        return copy.deepcopy(self.config)

    def save_to_file(self, file_path):
        with open(file_path, "w") as f:
            yaml.dump(self.config, f, default_flow_style=False)


DITANGO_CONFIG = None


def init_config(config_path=None, **overrides):
    global DITANGO_CONFIG
    DITANGO_CONFIG = DiTangoConfig(config_path=config_path, **overrides)
    return DITANGO_CONFIG


def get_config():
    return DITANGO_CONFIG


def print_config():
    cfg = get_config()
    if cfg is not None and cfg.rank == 0:
        print("\n===== DiTango Configuration =====", flush=True)
        for key, value in cfg.to_dict().items():
            print(f"{key}: {value}", flush=True)
