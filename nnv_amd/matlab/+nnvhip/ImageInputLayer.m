classdef ImageInputLayer < ImageInputLayer & nnvhip.RowMapLayer
    % ImageInputLayer whose normalisation of an ImageStar (ImageInputLayer.m:121-166) runs on the
    % device: every branch is a chain of centre offsets and whole-set scalings.
    methods
        function obj = ImageInputLayer(varargin)
            obj = obj@ImageInputLayer(varargin{:});
        end
        function [ops, scopes, params] = row_program(obj, h, w, c, ~)
            pr = @(a) nnvhip.RowMapLayer.per_row(a, h, w, c);
            hasRange = ~isempty(obj.Min) && ~isempty(obj.Max);
            switch obj.Normalization
                case 'none'
                    ops = []; scopes = []; params = [];
                case 'zerocenter'
                    ops = 0; scopes = 0; params = pr(-obj.Mean);
                case 'zscore'
                    ops = [0 3]; scopes = [0 1]; params = [pr(-obj.Mean), pr(obj.StandardDeviation(:))];
                case 'rescale-zero-one'
                    if hasRange
                        ops = [0 2]; scopes = [0 1]; params = [pr(-obj.Min), pr(1.0 / (obj.Max - obj.Min))];
                    else
                        ops = 2; scopes = 1; params = pr(1/255);
                    end
                case 'rescale-symmetric'
                    if hasRange
                        ops = [0 2 0]; scopes = [0 1 0]; params = [pr(-obj.Min), pr(2.0 / (obj.Max - obj.Min)), pr(-1)];
                    else
                        ops = [2 0]; scopes = [1 0]; params = [pr(2/255), pr(-1)];
                    end
                otherwise
                    error('The normalization method is not supported yet.');
            end
        end
        function images = reach_star_multipleInputs(obj, in_images, option) %#ok<INUSD>
            for i = 1:length(in_images)
                if ~isa(in_images(i), 'ImageStar'), error('Input is not an ImageStar'); end
            end
            images = obj.apply_rowmap(in_images);
        end
        function image = reach_star_single_input(obj, in_image)
            image = obj.reach_star_multipleInputs(in_image, 'single');
        end
    end
end
