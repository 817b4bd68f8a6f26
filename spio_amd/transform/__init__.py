"""Model conversion: replace matching nn.Conv2d modules with Conv2dGw8."""

from ._transform import transform, scan_modules, count_replaceable
