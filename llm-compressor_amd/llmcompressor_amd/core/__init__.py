"""Session, lifecycle, state and events (reference: src/llmcompressor/core/)."""
from __future__ import annotations

import threading
from dataclasses import dataclass, field
from enum import Enum, unique
from typing import Any, List, Optional

__all__ = ["EventType", "Event", "State", "CompressionLifecycle", "CompressionSession", "active_session",
           "create_session", "reset_session", "LifecycleCallbacks", "callbacks"]


@unique
class EventType(Enum):
    INITIALIZE = "initialize"
    FINALIZE = "finalize"
    BATCH_START = "batch_start"
    LOSS_CALCULATED = "loss_calculated"
    BATCH_END = "batch_end"
    CALIBRATION_START = "calibration_start"
    CALIBRATION_END = "calibration_end"
    SEQUENTIAL_EPOCH_END = "sequential_epoch_end"
    CALIBRATION_EPOCH_START = "calibration_epoch_start"
    CALIBRATION_EPOCH_END = "calibration_epoch_end"
    OPTIM_PRE_STEP = "optim_pre_step"
    OPTIM_POST_STEP = "optim_post_step"


@dataclass
class Event:
    type_: Optional[EventType] = None
    steps_per_epoch: Optional[int] = None
    batches_per_step: Optional[int] = None
    invocations_per_step: int = 1
    global_step: int = 0
    global_batch: int = 0

    @property
    def current_index(self) -> float:
        if not self.steps_per_epoch:
            return float(self.global_step)
        return self.global_step / self.steps_per_epoch


@dataclass
class State:
    model: Any = None
    teacher_model: Any = None
    optimizer: Any = None
    optim_wrapped: Optional[bool] = None
    loss: Any = None
    batch_data: Any = None
    data: dict = field(default_factory=dict)
    hardware: dict = field(default_factory=dict)
    loggers: Any = None
    model_log_cadence: Optional[float] = None
    sequential_prefetch: bool = False
    enable_compile: bool = False

    def update(self, model=None, calib_data=None, **kwargs):
        if model is not None:
            self.model = model
        if calib_data is not None:
            self.data["calib"] = calib_data
        for k, v in kwargs.items():
            if hasattr(self, k) and v is not None:
                setattr(self, k, v)
        return {}


@dataclass
class CompressionLifecycle:
    state: State = field(default_factory=State)
    recipe: Any = None
    initialized_: bool = False
    finalized: bool = False
    _last_event_type: Optional[EventType] = EventType.BATCH_END
    global_step: int = 0

    def reset(self):
        if self.recipe is not None:
            for mod in self.recipe.modifiers:
                if not mod.initialized or mod.finalized:
                    continue
                try:
                    mod.finalize(self.state)
                except Exception:
                    pass
        self.__init__()

    def initialize(self, recipe=None, recipe_stage=None, recipe_args=None, **kwargs) -> List[Any]:
        from ..recipe import Recipe

        self.state.update(**kwargs)
        if self.initialized_:
            return []
        self.recipe = Recipe.create_instance(recipe, modifier_group_name=recipe_stage) if recipe is not None else Recipe()
        out = []
        for mod in self.recipe.modifiers:
            out.append(mod.initialize(state=self.state, **kwargs))
        self.initialized_ = True
        return out

    def finalize(self, **kwargs) -> List[Any]:
        if not self.initialized_:
            raise ValueError("Cannot finalize before initializing")
        if self.finalized:
            raise ValueError("Cannot finalize more than once")
        out = [mod.finalize(state=self.state, **kwargs) for mod in self.recipe.modifiers]
        self.finalized = True
        return out

    def event(self, event_type: EventType, global_step: Optional[int] = 0, **kwargs) -> List[Any]:
        if not self.initialized_:
            raise ValueError("Cannot invoke event before initializing")
        if self.finalized:
            raise ValueError("Cannot invoke event after finalizing")
        if event_type in (EventType.INITIALIZE, EventType.FINALIZE):
            raise ValueError("Cannot invoke initialize or finalize events; use the corresponding methods")
        if event_type == EventType.LOSS_CALCULATED and (kwargs.get("loss") is None):
            raise ValueError("Loss must be provided for loss calculated event")
        if global_step is not None:
            self.global_step = global_step
        event = Event(type_=event_type, global_step=self.global_step)
        out = []
        for mod in self.recipe.modifiers:
            out.append(mod.update_event(state=self.state, event=event, **kwargs))
        return out


class CompressionSession:
    def __init__(self):
        self._lifecycle = CompressionLifecycle()

    @property
    def lifecycle(self) -> CompressionLifecycle:
        return self._lifecycle

    @property
    def state(self) -> State:
        return self._lifecycle.state

    def initialize(self, recipe=None, recipe_stage=None, recipe_args=None, model=None, calib_data=None, **kwargs):
        self._lifecycle.initialize(recipe=recipe, recipe_stage=recipe_stage, recipe_args=recipe_args, model=model,
                                   calib_data=calib_data, **kwargs)
        return self

    def finalize(self, **kwargs):
        return self._lifecycle.finalize(**kwargs)

    def event(self, event_type: EventType, batch_data=None, loss=None, **kwargs):
        return self._lifecycle.event(event_type=event_type, batch_data=batch_data, loss=loss, **kwargs)

    def reset(self):
        self._lifecycle.reset()

    def get_modifiers(self):
        return list(self._lifecycle.recipe.modifiers) if self._lifecycle.recipe is not None else []


_local = threading.local()
_global_session = CompressionSession()


def create_session() -> CompressionSession:
    _local.session = CompressionSession()
    return _local.session


def active_session() -> CompressionSession:
    return getattr(_local, "session", None) or _global_session


def reset_session():
    active_session().reset()


class LifecycleCallbacks:
    """Pipelines drive modifiers through these (reference: core/session_functions.py:55-175)."""

    @classmethod
    def event(cls, event_type: EventType, **kwargs):
        return active_session().event(event_type, **kwargs)

    @classmethod
    def batch_start(cls, batch_data=None, **kwargs):
        return cls.event(EventType.BATCH_START, batch_data=batch_data, **kwargs)

    @classmethod
    def batch_end(cls, **kwargs):
        return cls.event(EventType.BATCH_END, **kwargs)

    @classmethod
    def calibration_start(cls, **kwargs):
        return cls.event(EventType.CALIBRATION_START, **kwargs)

    @classmethod
    def sequential_epoch_end(cls, modules, **kwargs):
        return cls.event(EventType.SEQUENTIAL_EPOCH_END, modules=modules, **kwargs)

    @classmethod
    def calibration_epoch_start(cls, **kwargs):
        return cls.event(EventType.CALIBRATION_EPOCH_START, **kwargs)

    @classmethod
    def calibration_epoch_end(cls, **kwargs):
        return cls.event(EventType.CALIBRATION_EPOCH_END, **kwargs)

    @classmethod
    def calibration_end(cls, **kwargs):
        return cls.event(EventType.CALIBRATION_END, **kwargs)


callbacks = LifecycleCallbacks
