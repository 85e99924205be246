"""Sparsity logger with the reference's files and schema, without its per-layer host synchronisation.

reference: src/psa_triton/utils/psa_logger.py:13-537 (PSALogger).  A session directory holds
    config.json     session name, time stamp, model type, layer / inference counts, the attention configuration
    sparsity.jsonl  one line per layer call: global_step, timestamp, layer_idx, sparsity, density, per_head_density,
                    sequence_length, batch_size, num_heads, is_warmup, use_sim_mask, sim_mask_stats{pool_Nx_ratio}
    summary.txt     per-layer table (count, mean, min, max, standard deviation), overall and non-warm-up statistics,
                    and the average distribution of the similarity cap over the pooling levels
The reference brings every value to the host when it is logged (`.cpu()` / `.item()` per layer).  Here sparsity,
per-head density and the similarity-cap histogram may be device tensors: they are queued and only read when the queue
is flushed (every `flush_every` records, on write_summary() and on close()), so a layer call does not wait for the GPU.
"""
import json
from dataclasses import asdict
from datetime import datetime
from pathlib import Path
from typing import Any, Dict, List, Optional

import torch

LEVELS = (1, 2, 4, 8)


def sim_mask_ratios(sim_mask: Optional[torch.Tensor]):
    """Share of the kv-blocks whose similarity cap is 1, 2, 4, 8: a 4-element tensor on sim_mask's device (no
    synchronisation), or None without a cap.  reference: psa_logger.py:140-177."""
    if sim_mask is None:
        return None
    flat = sim_mask.reshape(-1)
    n = max(flat.numel(), 1)
    return torch.stack([(flat == lv).sum() for lv in LEVELS]).to(torch.float32) / n


class PSALogger:
    def __init__(self, log_dir: str, config: Any, model_type: str = "wan", layer_num: int = 42, inference_num: int = 50,
                 session_name: Optional[str] = None, flush_every: int = 256):
        self.log_dir = Path(log_dir)
        self.log_dir.mkdir(parents=True, exist_ok=True)
        self.config, self.model_type, self.layer_num, self.inference_num = config, model_type, layer_num, inference_num
        self.session_name = session_name or "psa_session_" + datetime.now().strftime("%Y%m%d_%H%M%S")
        self.session_dir = self.log_dir / self.session_name
        self.session_dir.mkdir(parents=True, exist_ok=True)
        self.config_file = self.session_dir / "config.json"
        self.sparsity_file = self.session_dir / "sparsity.jsonl"
        self.summary_file = self.session_dir / "summary.txt"
        self.sparsity_handle = open(self.sparsity_file, "a", encoding="utf-8")
        self.layer_stats: Dict[int, Dict[str, Any]] = {}
        self.global_counter = 0
        self.flush_every = flush_every
        self._pending: List[dict] = []
        self._write_config()

    # ------------------------------------------------------------------ files
    def _write_config(self):
        cfg = self.config
        if hasattr(cfg, "__dataclass_fields__"):
            cfg = {k: ({str(a): list(b) for a, b in v.items()} if isinstance(v, dict) else v) for k, v in asdict(cfg).items()}
        else:
            cfg = str(cfg)
        with open(self.config_file, "w", encoding="utf-8") as f:
            json.dump({"session_name": self.session_name, "timestamp": datetime.now().isoformat(), "model_type": self.model_type,
                       "layer_num": self.layer_num, "inference_num": self.inference_num, "config": cfg}, f, indent=2)

    # ------------------------------------------------------------------ logging
    def log_sparsity(self, layer_idx: int, sparsity, per_head_density, sequence_length: int, batch_size: int = 1,
                     num_heads: int = -1, sim_mask: Optional[torch.Tensor] = None, is_warmup: bool = False):
        """Queue one record.  sparsity / per_head_density may be Python numbers / lists or device tensors; sim_mask is
        the similarity cap [B, H, Nk] (values 1, 2, 4, 8) or None."""
        self.global_counter += 1
        self._pending.append(dict(global_step=self.global_counter, timestamp=datetime.now().isoformat(), layer_idx=layer_idx,
                                  sparsity=sparsity, per_head_density=per_head_density, sequence_length=sequence_length,
                                  batch_size=batch_size, num_heads=num_heads, is_warmup=is_warmup, sim=sim_mask_ratios(sim_mask)))
        if len(self._pending) >= self.flush_every:
            self.flush()

    def _new_layer(self):
        inf = float("inf")
        return {"count": 0, "total_sparsity": 0.0, "min_sparsity": inf, "max_sparsity": 0.0, "sparsity_history": [],
                "non_warmup_count": 0, "non_warmup_total_sparsity": 0.0, "non_warmup_min_sparsity": inf,
                "non_warmup_max_sparsity": 0.0, "non_warmup_sparsity_history": [],
                "sim_mask_stats": {"pool_1x_sum": 0.0, "pool_2x_sum": 0.0, "pool_4x_sum": 0.0, "pool_8x_sum": 0.0, "count": 0}}

    def flush(self):
        """Read the queued values (this is where the host waits for the GPU), update the statistics, write the lines."""
        if not self._pending or self.sparsity_handle is None:
            return
        sim_enabled = bool(getattr(self.config, "use_sim_mask", True))
        for rec in self._pending:
            sp = float(rec["sparsity"])
            ph = rec["per_head_density"]
            ph = [float(x) for x in (ph.detach().cpu().reshape(-1).tolist() if torch.is_tensor(ph) else ph)]
            sim = rec["sim"]
            ratios = [float(x) for x in sim.cpu().tolist()] if sim is not None else [0.0, 0.0, 0.0, 0.0]
            st = self.layer_stats.setdefault(rec["layer_idx"], self._new_layer())
            st["count"] += 1
            st["total_sparsity"] += sp
            st["min_sparsity"] = min(st["min_sparsity"], sp)
            st["max_sparsity"] = max(st["max_sparsity"], sp)
            st["sparsity_history"] = (st["sparsity_history"] + [sp])[-100:]
            if sp > 0:  # a dense (warm-up) call has sparsity 0
                st["non_warmup_count"] += 1
                st["non_warmup_total_sparsity"] += sp
                st["non_warmup_min_sparsity"] = min(st["non_warmup_min_sparsity"], sp)
                st["non_warmup_max_sparsity"] = max(st["non_warmup_max_sparsity"], sp)
                st["non_warmup_sparsity_history"] = (st["non_warmup_sparsity_history"] + [sp])[-100:]
            if sim_enabled and not rec["is_warmup"] and sim is not None:
                for name, r in zip(("pool_1x_sum", "pool_2x_sum", "pool_4x_sum", "pool_8x_sum"), ratios):
                    st["sim_mask_stats"][name] += r
                st["sim_mask_stats"]["count"] += 1
            entry = {
                "global_step": rec["global_step"], "timestamp": rec["timestamp"], "layer_idx": rec["layer_idx"],
                "sparsity": round(sp, 6), "density": round(1 - sp, 6), "per_head_density": [round(d, 6) for d in ph],
                "sequence_length": rec["sequence_length"], "batch_size": rec["batch_size"],
                "num_heads": rec["num_heads"] if rec["num_heads"] > 0 else len(ph), "is_warmup": bool(rec["is_warmup"]),
                "use_sim_mask": sim_enabled,
                "sim_mask_stats": {"pool_%dx_ratio" % lv: round(r, 6) for lv, r in zip(LEVELS, ratios)},
            }
            self.sparsity_handle.write(json.dumps(entry) + "\n")
        self.sparsity_handle.flush()
        self._pending = []

    # ------------------------------------------------------------------ summary
    @staticmethod
    def _std(xs):
        if len(xs) < 2:
            return 0.0
        m = sum(xs) / len(xs)
        return (sum((x - m) ** 2 for x in xs) / len(xs)) ** 0.5

    def write_summary(self):
        self.flush()
        if not self.layer_stats:
            return
        bar, rule = "=" * 80, "-" * 80
        out = ["", bar, "PSA Sparsity Summary - %s" % self.session_name, bar,
               "Generated: %s" % datetime.now().strftime("%Y-%m-%d %H:%M:%S"), "Total Forward Passes: %d" % self.global_counter, "",
               "Per-Layer Statistics:", rule,
               "%-8s %-8s %-15s %-10s %-10s %-10s" % ("Layer", "Count", "Avg Sparsity", "Min", "Max", "StdDev"), rule]
        for idx in sorted(self.layer_stats):
            st = self.layer_stats[idx]
            out.append("%-8d %-8d %-15.6f %-10.6f %-10.6f %-10.6f" % (idx, st["count"], st["total_sparsity"] / st["count"],
                                                                   st["min_sparsity"], st["max_sparsity"], self._std(st["sparsity_history"])))
        out += [rule, "", "Overall Statistics:", rule]
        hist = [x for st in self.layer_stats.values() for x in st["sparsity_history"]]
        count = sum(st["count"] for st in self.layer_stats.values())
        total = sum(st["total_sparsity"] for st in self.layer_stats.values())
        if hist:
            out += ["Average Sparsity (all layers): %.6f" % (total / count), "Average Density (all layers): %.6f" % (1 - total / count),
                    "Sparsity Range: [%.6f, %.6f]" % (min(hist), max(hist)), "Standard Deviation: %.6f" % self._std(hist),
                    "Total Samples: %d" % len(hist)]
        out += ["", "Non-Warmup Statistics (excluding density=1.0 steps):", rule]
        nw = [x for st in self.layer_stats.values() for x in st["non_warmup_sparsity_history"]]
        nw_count = sum(st["non_warmup_count"] for st in self.layer_stats.values())
        nw_total = sum(st["non_warmup_total_sparsity"] for st in self.layer_stats.values())
        if nw:
            out += ["Average Sparsity (non-warmup): %.6f" % (nw_total / nw_count),
                    "Average Density (non-warmup): %.6f" % (1 - nw_total / nw_count),
                    "Sparsity Range: [%.6f, %.6f]" % (min(nw), max(nw)), "Standard Deviation: %.6f" % self._std(nw),
                    "Non-Warmup Samples: %d" % len(nw), "Warmup Samples (density=1.0): %d" % (count - nw_count)]
        else:
            out.append("No non-warmup samples recorded (all steps were warmup).")
        if bool(getattr(self.config, "use_sim_mask", True)):
            out += ["", "Sim Mask Statistics (Average Pooling Distribution):", rule,
                    "%-8s %-12s %-12s %-12s %-12s" % ("Layer", "1x Pool %", "2x Pool %", "4x Pool %", "8x Pool %"), rule]
            tot, n_all = [0.0] * 4, 0
            for idx in sorted(self.layer_stats):
                sm = self.layer_stats[idx]["sim_mask_stats"]
                if sm["count"] > 0:
                    sums = [sm["pool_%dx_sum" % lv] for lv in LEVELS]
                    out.append("%-8d " % idx + " ".join("%-12.2f" % (s / sm["count"] * 100) for s in sums))
                    tot = [a + b for a, b in zip(tot, sums)]
                    n_all += sm["count"]
            out.append(rule)
            if n_all > 0:
                pct = [t / n_all * 100 for t in tot]
                out.append("%-8s " % "Overall" + " ".join("%-12.2f" % x for x in pct))
                out += ["", "Overall Pooling Distribution (all layers average):",
                        "  1x Pooling (no pooling):  %.2f%%" % pct[0], "  2x Pooling:               %.2f%%" % pct[1],
                        "  4x Pooling:               %.2f%%" % pct[2], "  8x Pooling:               %.2f%%" % pct[3],
                        "  Total:                    %.2f%%" % sum(pct), "  Total Sim Mask Samples:   %d" % n_all]
        else:
            out += ["", "Sim Mask Statistics: disabled (use_sim_mask = False)", rule]
        out += [bar, ""]
        with open(self.summary_file, "a", encoding="utf-8") as f:
            f.write("\n".join(out))

    def close(self):
        if self.sparsity_handle is not None:
            self.flush()
            self.sparsity_handle.close()
            self.sparsity_handle = None
            self.write_summary()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
