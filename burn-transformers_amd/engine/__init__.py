from .plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry

__all__ = ["LayerPlan", "ModelPlan", "PartSpec", "ScheduleEntry"]
