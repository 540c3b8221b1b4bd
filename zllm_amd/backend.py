"""The backends zllm runs on (src/backend/backend.zig:13-19), with the member
this package adds."""
import enum


class Backend(enum.Enum):
    webgpu = 0
    agility = 1
    hip = 2
