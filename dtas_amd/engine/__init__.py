from .database import DataBase
from .tuner import Engine
