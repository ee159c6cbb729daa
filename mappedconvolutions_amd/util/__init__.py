from .point_functions import knn
from .spherical_projections import (get_projection_map, get_perspective_projection_map,
                                    get_reverse_cube_projection_map, cube_to_rect)
from .icosphere_functions import (convert_3d_to_spherical, gnomonic_kernel,
                                  kernel_map_from_samples, vertex_to_vertex_kernel_map)
from .synthetic import (latitude_map, cube_to_equirect_map, mesh_weighted_map, sphere_points)

__all__ = ['knn', 'convert_3d_to_spherical', 'gnomonic_kernel', 'kernel_map_from_samples',
           'vertex_to_vertex_kernel_map', 'get_projection_map', 'get_perspective_projection_map',
           'get_reverse_cube_projection_map', 'cube_to_rect', 'latitude_map', 'cube_to_equirect_map', 'mesh_weighted_map', 'sphere_points']
