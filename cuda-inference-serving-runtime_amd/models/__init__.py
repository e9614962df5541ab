from .model import Model, ScheduleEntry
from .llama import build_llama
from .novosun import build_novosun
from .ditazen import build_ditazen
from .noresun import build_noresun
from .zovozen import build_zovozen
