"""qconfig JSON schema: QLinearConfig -> Expert{gate, up, down} -> Layer{experts} -> Model{layers}.

Same classes, field names, defaults and JSON shape as the reference (mxmoe/kernels/qconfig.py:6-106), so a qconfig
written by the reference's ILP (`export_qconfig`, mxmoe/quant/bits_solver.py:25-71) loads unchanged.
"""
from __future__ import annotations

import dataclasses
import json


@dataclasses.dataclass
class QLinearConfig:
    w_bits: int = 16
    w_gsize: int = -1
    w_sym: bool = False
    w_clip: tuple = (1.0, 1.0)
    a_bits: int = 16
    a_gsize: int = -1
    a_sym: bool = True
    a_clip: tuple = (1.0, 1.0)

    def __str__(self):
        return f"W{self.w_bits}A{self.a_bits}_g{self.w_gsize}_{'sym' if self.w_sym else 'asym'}"

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @staticmethod
    def from_dict(d: dict) -> "QLinearConfig":
        return QLinearConfig(**{f.name: d[f.name] for f in dataclasses.fields(QLinearConfig)})

    def qparams(self) -> tuple:
        """(a_bits, w_bits, gsize, sym): the tuple the operators take per expert (ref_bind.cu:321,365)."""
        return (self.a_bits, self.w_bits, self.w_gsize, bool(self.w_sym))


@dataclasses.dataclass
class QExpertConfig:
    gate: QLinearConfig
    up: QLinearConfig
    down: QLinearConfig

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    def qmap(self) -> dict:
        return {"gate": self.gate, "up": self.up, "down": self.down}


@dataclasses.dataclass
class QLayerConfig:
    experts: dict

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)


@dataclasses.dataclass
class QModelConfig:
    layers: dict

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)


def build_qmodel_cfg_from_dict(cfg: dict) -> QModelConfig:
    cfg = dict(cfg)
    cfg.pop("LT", None)
    layers = {}
    for layer_idx, layer_cfg in cfg.items():
        experts = {}
        for expert_idx, ecfg in layer_cfg["experts"].items():
            experts[expert_idx] = QExpertConfig(gate=QLinearConfig(**ecfg["gate"]), up=QLinearConfig(**ecfg["up"]), down=QLinearConfig(**ecfg["down"]))
        layers[layer_idx] = QLayerConfig(experts=experts)
    return QModelConfig(layers=layers)


def build_qmodel_cfg_from_json(json_path: str) -> QModelConfig:
    with open(json_path, "r") as f:
        return build_qmodel_cfg_from_dict(json.load(f))


def build_uni_qexpert_cfg(qcfg: QLinearConfig) -> QExpertConfig:
    return QExpertConfig(gate=qcfg, up=qcfg, down=qcfg)


def build_uni_qlayer_cfg(qcfg: QLinearConfig, num_experts: int) -> QLayerConfig:
    return QLayerConfig(experts={str(i): build_uni_qexpert_cfg(qcfg) for i in range(num_experts)})


def build_uni_qmodel_cfg(qcfg: QLinearConfig, num_layers: int, num_experts: int) -> QModelConfig:
    return QModelConfig(layers={str(i): build_uni_qlayer_cfg(qcfg, num_experts) for i in range(num_layers)})


def get_all_wbits(qmodel_cfg: QModelConfig) -> list:
    bits = set()
    for layer in qmodel_cfg.layers.values():
        for expert in layer.experts.values():
            for q in expert.qmap().values():
                bits.add((q.w_bits, q.w_gsize, q.w_sym))
    return list(bits)
