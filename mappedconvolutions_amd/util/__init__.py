from .point_functions import knn
from .synthetic import (latitude_map, cube_to_equirect_map, mesh_weighted_map, sphere_points)

__all__ = ['knn', 'latitude_map', 'cube_to_equirect_map', 'mesh_weighted_map', 'sphere_points']
