from .step import AttentionPlan, KVView, SeqStep, StepContext
