from ..registry import register_op

register_hip_op = register_op("hip")
