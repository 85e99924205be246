"""Preset loader: attention_config.yaml -> keyword arguments of AttentionConfig.

Follows the reference loader field by field, including its defaults
(reference: modify_diffusers.py:39-178, WanAttentionConfigLoader)."""
import math
import os
from pathlib import Path
from typing import Any, Dict, List, Optional, Tuple, Union

import yaml

DEFAULT_CONFIG = Path(__file__).parent / "configs" / "attention_config.yaml"


class AttentionConfigLoader:
    def __init__(self, config_path: Optional[str] = None):
        path = Path(config_path) if config_path is not None else DEFAULT_CONFIG
        if not path.exists():
            raise FileNotFoundError(f"Config file not found: {path}")
        with open(path, "r", encoding="utf-8") as f:
            self._config = yaml.safe_load(f) or {}

    def _model(self, model_name: str) -> Dict[str, Any]:
        cfg = self._config.get(model_name)
        if cfg is None:
            raise ValueError(f"Model '{model_name}' not found in config. Available models: {list(self._config.keys())}")
        return cfg

    def list_presets(self, model_name: str) -> List[str]:
        return list(self._model(model_name).get("attention_configs", {}).keys())

    def get_attention_config(self, model_name: str, preset_name: Optional[str],
                             video_shape: Union[List[int], Tuple[int, int, int]]) -> Dict[str, Any]:
        """-> {name, type, description, video_dims, original_video_shape[, params]}; `params` feeds
        AttentionConfig(**params).  video_shape = [width, height, depth] in pixels / frames."""
        model_cfg = self._model(model_name)
        presets = model_cfg.get("attention_configs", {})
        if not presets:
            raise ValueError(f"No attention presets defined for model '{model_name}'.")
        if preset_name is None:
            preset_name = model_cfg.get("default_attention")
        if preset_name is None:
            raise ValueError(f"Preset name must be provided for model '{model_name}'. Available presets: {list(presets.keys())}")
        if preset_name not in presets:
            raise ValueError(f"Preset '{preset_name}' not found for model '{model_name}'. Available presets: {list(presets.keys())}")
        pc = presets[preset_name]
        ptype = pc.get("type", "psa").lower()
        if video_shape is None or len(video_shape) != 3:
            raise ValueError("video_shape must be a sequence of [width, height, depth].")
        vs = [int(video_shape[0]), int(video_shape[1]), int(video_shape[2])]
        if "video_scale" not in model_cfg:
            raise ValueError("Missing 'video_scale' configuration for model.")
        sc = model_cfg["video_scale"]
        dims = {
            "width": math.ceil(vs[0] / sc["width_divisor"]),
            "height": math.ceil(vs[1] / sc["height_divisor"]),
            "depth": math.ceil(vs[2] / sc["depth_divisor"]),
        }
        info: Dict[str, Any] = {
            "name": preset_name,
            "type": ptype,
            "description": pc.get("description"),
            "video_dims": dims,
            "original_video_shape": {"width": vs[0], "height": vs[1], "depth": vs[2]},
        }
        if ptype == "dense":
            return info
        if ptype != "psa":
            raise ValueError(f"Unsupported preset type '{ptype}' for model '{model_name}'.")
        blk = pc.get("block_size", {})
        tile_size = pc.get("tile_size")
        params: Dict[str, Any] = {
            **dims,
            "text_length": pc.get("text_length", model_cfg.get("text_length", 0)),
            "use_rearrange": pc.get("use_rearrange", True),
            "use_sim_mask": pc.get("use_sim_mask", True),
            "block_m": blk.get("m", 128),
            "block_n": blk.get("n", 128),
            "tile_n": blk.get("tile_n", 32),
            "mask_ratios": {int(k): tuple(v) for k, v in pc.get("mask_ratios", {}).items()},
            "mask_mode": pc.get("mask_mode", "thresholdbound"),
            "attn_impl": pc.get("attn_impl", "new_mask_type"),
            "warmup_steps": pc.get("warmup_steps", 0),
            "tile_size": tuple(tile_size) if tile_size is not None else None,
            "rearrange_method": pc.get("rearrange_method", "Gilbert"),
            "verbose": pc.get("verbose", False),
            "enable_logging": pc.get("enable_logging", True),
            "log_dir": pc.get("log_dir", "./psa_logs/"),
        }
        for key in ("sim_2x_threshold", "sim_4x_threshold", "sim_8x_threshold"):
            if key in pc:
                params[key] = pc[key]
        st = pc.get("sim_thresholds", {})
        if st:
            params.setdefault("sim_2x_threshold", st.get("x2"))
            params.setdefault("sim_4x_threshold", st.get("x4"))
            params.setdefault("sim_8x_threshold", st.get("x8"))
        info["params"] = params
        return info
