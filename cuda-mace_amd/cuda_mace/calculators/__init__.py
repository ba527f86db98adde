from .device_calculator import DeviceCalculator  # noqa: F401
