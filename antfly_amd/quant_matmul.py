"""Quant-matmul dispatch vocabulary, mirroring graph/quant_matmul.zig of the
reference (enums :17-55, Shape/Plan :216-232, plan/select :241-268, rowBucket
:558-564).  The decisions themselves are made by the C ABI."""
from __future__ import annotations

import enum
from dataclasses import dataclass

from . import _lib


class DispatchKind(enum.IntEnum):
    scalar = 0
    mmv = 1
    small_batch = 2
    mm = 3


class Primitive(enum.IntEnum):
    mat_vec = 0
    mat_vec_ext = 1
    mat_mat = 2
    scalar = 3


class Operator(enum.IntEnum):
    fallback = 0
    mul_mv = 1
    mul_mv_ext = 2
    mul_mm = 3
    get_rows = 4


class RowBucket(enum.IntEnum):
    rows_0 = 0
    rows_1 = 1
    rows_2_8 = 2
    rows_9_64 = 3
    rows_65_plus = 4


class Format(enum.IntEnum):
    unknown = 0
    q4_0 = 1
    q8_0 = 5
    q4_k = 9
    f32 = 254


@dataclass
class Shape:
    rows: int
    in_dim: int
    out_dim: int
    format: Format


@dataclass
class Plan:
    dispatch: DispatchKind
    primitive: Primitive
    operator: Operator
    row_bucket: RowBucket
    format: Format
    rows: int
    in_dim: int
    out_dim: int

    def to_c(self) -> "_lib.QuantPlan":
        return _lib.QuantPlan(int(self.dispatch), int(self.primitive), int(self.operator), int(self.row_bucket),
                              int(self.format), self.rows, self.in_dim, self.out_dim)


def select(shape: Shape) -> DispatchKind:
    return DispatchKind(_lib.lib().afhip_quant_matmul_select(shape.rows, shape.in_dim, shape.out_dim, int(shape.format)))


def plan(shape: Shape) -> Plan:
    p = _lib.QuantPlan()
    _lib.lib().afhip_quant_matmul_plan(shape.rows, shape.in_dim, shape.out_dim, int(shape.format), p)
    return Plan(DispatchKind(p.dispatch), Primitive(p.primitive), Operator(p.op), RowBucket(p.row_bucket),
                Format(p.format), p.rows, p.in_dim, p.out_dim)


def q8_0(rows: int, in_dim: int, out_dim: int) -> Plan:
    return plan(Shape(rows, in_dim, out_dim, Format.q8_0))


def rowBucket(rows: int) -> RowBucket:
    return RowBucket(_lib.lib().afhip_quant_row_bucket(rows))


def formatFromTensorType(tensor_type: int) -> Format:
    return Format(_lib.lib().afhip_quant_format_from_tensor_type(tensor_type))


class OperatorPlanKind(enum.IntEnum):
    quant_matmul = 0
    quant_row = 1
    attention = 2


@dataclass
class OperatorPlan:
    """graph/operator_plan.zig:24-38: tagged union; only quant_matmul carries data here."""

    kind: OperatorPlanKind
    quant_matmul: Plan | None = None

    def to_c(self) -> "_lib.OperatorPlan":
        qp = self.quant_matmul.to_c() if self.quant_matmul is not None else _lib.QuantPlan()
        return _lib.OperatorPlan(int(self.kind), qp)
